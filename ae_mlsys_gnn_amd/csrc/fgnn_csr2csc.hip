// GPU CSR -> CSC transpose (stable), replacing the reference's cuSPARSE call
// (src/csr2csc/csr2csc.cu:10-23).
//
// The transpose is a stable sort of the CSR positions by column: an LSD radix sort with digits of
// up to 8 bits over key = col_ind[p], payload = p.  Each pass is histogram -> scan -> stable scatter:
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

__global__ __launch_bounds__(RS_TPB) void rs_hist_kernel(const int *__restrict__ keys, int64_t n, int shift, int mask, int nblocks, int *__restrict__ hist)
{
    __shared__ int cnt[4][256];         // one set of counters per wave: a quarter of the collisions
    for (int i = (int)threadIdx.x; i < 4 * 256; i += RS_TPB) (&cnt[0][0])[i] = 0;
    __syncthreads();
    const int wave = fg_wave(), lane = fg_lane();
#pragma unroll 4
    for (int it = 0; it < RS_ITEMS; ++it) {
        int64_t i = (int64_t)blockIdx.x * RS_TILE + wave * RS_SUB + it * 64 + lane;
        if (i < n) atomicAdd(&cnt[wave][(keys[i] >> shift) & mask], 1);
    }
    __syncthreads();
    if ((int)threadIdx.x <= mask)
        hist[(size_t)threadIdx.x * nblocks + blockIdx.x] = (cnt[0][threadIdx.x] + cnt[1][threadIdx.x]) + (cnt[2][threadIdx.x] + cnt[3][threadIdx.x]);
}

// One workgroup per digit: exclusive scan of that digit's per-block counts in place.  The row is walked
// in chunks of RS_TPB * 8 counts: every thread scans 8 consecutive counts serially, the 256 thread totals
// are scanned with wave shuffles and one exchange through LDS, and the chunk's total carries over.
__global__ __launch_bounds__(RS_TPB) void rs_scan_kernel(int *__restrict__ hist, int nblocks, int *__restrict__ digit_total)
{
    constexpr int PER = 8;
    __shared__ int wave_tot[4];
    int *row = hist + (size_t)blockIdx.x * nblocks;
    const int lane = fg_lane(), wave = fg_wave();
    int carry = 0;
    for (int base = 0; base < nblocks; base += RS_TPB * PER) {
        const int i0 = base + (int)threadIdx.x * PER;
        int v[PER], tot = 0;
#pragma unroll
        for (int j = 0; j < PER; ++j) { v[j] = i0 + j < nblocks ? row[i0 + j] : 0; tot += v[j]; }
        int incl = tot;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            int t = __shfl_up(incl, off);
            if (lane >= off) incl += t;
        }
        __syncthreads();                        // the previous chunk's wave totals have been read
        if (lane == 63) wave_tot[wave] = incl;
        __syncthreads();
        int run = carry + incl - tot;
        for (int w = 0; w < wave; ++w) run += wave_tot[w];
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            if (i0 + j < nblocks) row[i0 + j] = run;
            run += v[j];
        }
        carry += wave_tot[0] + wave_tot[1] + wave_tot[2] + wave_tot[3];
    }
    if (threadIdx.x == 0) digit_total[blockIdx.x] = carry;
}

__global__ __launch_bounds__(256) void rs_digit_base_kernel(const int *__restrict__ digit_total, int n_digits, int *__restrict__ digit_base)
{
    __shared__ int sh[256];
    int v = (int)threadIdx.x < n_digits ? digit_total[threadIdx.x] : 0;
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
// The tile is first sorted by digit inside LDS (local position = the digit's base inside the tile +
// rank among the tile's earlier elements of that digit), then written out in local order: all
// elements of a digit leave as one contiguous run, so neighbouring lanes write neighbouring addresses
// instead of 4-byte stores scattered over 256 destinations.
__global__ __launch_bounds__(RS_TPB) void rs_scatter_kernel(const int *__restrict__ keys_in, const int *__restrict__ pay_in, int64_t n, int shift,
                                                            int bits, int nblocks, const int *__restrict__ hist, const int *__restrict__ digit_base,
                                                            int *__restrict__ keys_out, int *__restrict__ pay_out)
{
    __shared__ int wcnt[4][256];        // per wave and digit: count, then the running local position
    __shared__ int gofs[256];           // per digit: global position of the tile's run minus its local base
    __shared__ int wave_tot[4];
    __shared__ int skey[RS_TILE], spay[RS_TILE];
    const int wave = fg_wave(), lane = fg_lane();
    const int mask = (1 << bits) - 1;
    for (int i = (int)threadIdx.x; i < 4 * 256; i += RS_TPB) (&wcnt[0][0])[i] = 0;
    __syncthreads();
    const int64_t tile0 = (int64_t)blockIdx.x * RS_TILE;
    int key[RS_ITEMS], pay[RS_ITEMS];
#pragma unroll
    for (int it = 0; it < RS_ITEMS; ++it) {
        int64_t i = tile0 + wave * RS_SUB + it * 64 + lane;
        key[it] = i < n ? keys_in[i] : 0;
        pay[it] = (pay_in && i < n) ? pay_in[i] : (int)i;      // fetched up front: the ranking loop below is a dependent chain
        if (i < n) atomicAdd(&wcnt[wave][(key[it] >> shift) & mask], 1);
    }
    __syncthreads();
    {
        // thread d owns digit d: exclusive scan of the tile's digit counts (inside the wave by shuffles,
        // across the four waves through LDS), then the per-wave starting positions
        const int d = (int)threadIdx.x;
        int c[4], tot = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) { c[w] = wcnt[w][d]; tot += c[w]; }
        int incl = tot;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            int t = __shfl_up(incl, off);
            if (lane >= off) incl += t;
        }
        if (lane == 63) wave_tot[wave] = incl;
        __syncthreads();
        int lbase = incl - tot;
        for (int w = 0; w < wave; ++w) lbase += wave_tot[w];
        gofs[d] = d <= mask ? digit_base[d] + hist[(size_t)d * nblocks + blockIdx.x] - lbase : 0;
        int run = lbase;
#pragma unroll
        for (int w = 0; w < 4; ++w) { wcnt[w][d] = run; run += c[w]; }
    }
    __syncthreads();
    const unsigned long long lt = (1ull << lane) - 1ull;
#pragma unroll
    for (int it = 0; it < RS_ITEMS; ++it) {
        int64_t i = tile0 + wave * RS_SUB + it * 64 + lane;
        bool ok = i < n;
        int d = (key[it] >> shift) & mask;
        unsigned long long peers = __builtin_amdgcn_ballot_w64(ok);
#pragma unroll
        for (int bit = 0; bit < 8; ++bit) {
            if (bit < bits) {
                unsigned long long bal = __builtin_amdgcn_ballot_w64(((d >> bit) & 1) != 0);
                peers &= ((d >> bit) & 1) ? bal : ~bal;
            }
        }
        int rank = __popcll(peers & lt);
        int base = wcnt[wave][d];
        if (ok) {
            skey[base + rank] = key[it];
            spay[base + rank] = pay[it];
        }
        fg_wave_lds_sync();
        // the highest lane of every peer group advances the wave's counter of that digit
        if (ok && (peers >> lane) == 1ull) wcnt[wave][d] = base + __popcll(peers);
        fg_wave_lds_sync();
    }
    __syncthreads();
    const int count = (int)((n - tile0) < (int64_t)RS_TILE ? (n - tile0) : (int64_t)RS_TILE);
#pragma unroll 4
    for (int i = (int)threadIdx.x; i < count; i += RS_TPB) {
        int k = skey[i];
        int dst = gofs[(k >> shift) & mask] + i;
        keys_out[dst] = k;
        pay_out[dst] = spay[i];
    }
}

// Row of CSR position p: the last r with row_ptr[r] <= p, searched in [lo, hi) with row_ptr[lo] <= p < row_ptr[hi].
__device__ __forceinline__ int csc_row_of(const int *__restrict__ row_ptr, int lo, int hi, int p)
{
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if (row_ptr[mid] <= p) lo = mid; else hi = mid;
    }
    return lo;
}

// hint[k] = row of position min(k << CSC_HINT_SHIFT, n - 1), k = 0 .. n_hint - 1: a coarse inverse of
// row_ptr, so that the per-entry search of csc_finalize_kernel covers the few rows of one bucket of
// positions instead of the whole pointer array.
#define CSC_HINT_SHIFT 9
__global__ __launch_bounds__(256) void csc_row_hint_kernel(int64_t n, int n_rows, int n_hint, const int *__restrict__ row_ptr, int *__restrict__ hint)
{
    int k = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (k >= n_hint) return;
    int64_t p = (int64_t)k << CSC_HINT_SHIFT;
    if (p > n - 1) p = n - 1;
    hint[k] = csc_row_of(row_ptr, 0, n_rows, (int)p);
}

__global__ __launch_bounds__(256) void csc_finalize_kernel(int64_t n, int n_cols, const int *__restrict__ sorted_keys,
                                                           const int *__restrict__ permute, const int *__restrict__ row_ptr,
                                                           const int *__restrict__ hint, int *__restrict__ col_ptr, int *__restrict__ row_ind)
{
    int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (q >= n) return;
    int key = sorted_keys[q];
    int prev = q > 0 ? sorted_keys[q - 1] : -1;
    for (int c = prev + 1; c <= key; ++c) col_ptr[c] = (int)q;
    if (q == n - 1)
        for (int c = key + 1; c <= n_cols; ++c) col_ptr[c] = (int)n;
    int p = permute[q];
    int k = p >> CSC_HINT_SHIFT;
    row_ind[q] = csc_row_of(row_ptr, hint[k], hint[k + 1] + 1, p);
}

__global__ __launch_bounds__(256) void fill_i32_kernel(int *p, size_t n, int v)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// Key bits to sort for ids below n_cols.
static int rs_key_bits(int n_cols)
{
    int bits = 1;
    while (bits < 31 && (1LL << bits) < (long long)n_cols) ++bits;
    return bits;
}

// Scratch of one radix sort of n (key, payload) pairs: two key buffers, one payload buffer,
// per-block digit counts and two 256-entry tables.
static size_t rs_sort_workspace(int64_t n)
{
    size_t nblocks = (size_t)((n + RS_TILE - 1) / RS_TILE);
    return 3 * fgnn_align256((size_t)n * sizeof(int)) + fgnn_align256(256 * nblocks * sizeof(int)) + 2 * fgnn_align256(256 * sizeof(int));
}

// Stable LSD radix sort of n pairs by the low `key_bits` key bits, in ceil(key_bits / 8) passes of equal
// digit width (18 bits: 6 + 6 + 6 rather than 8 + 8 + 2 -- fewer digits mean longer contiguous runs per
// tile in the scatter).  keys_in is not modified; pay_in == NULL sorts the element indices.  The sorted
// payload lands in pay_out; *sorted_keys points at the sorted keys (inside the workspace).
static int rs_sort_pairs(const int *keys_in, const int *pay_in, int64_t n, int key_bits, int *pay_out, const int **sorted_keys, void *workspace,
                         hipStream_t st)
{
    const int passes = (key_bits + 7) / 8;
    const int bits = (key_bits + passes - 1) / passes;      // digit width of every pass, <= 8
    const int nblocks = (int)((n + RS_TILE - 1) / RS_TILE);
    char *w = (char *)workspace;
    int *keys[2];
    keys[0] = (int *)w; w += fgnn_align256((size_t)n * sizeof(int));
    keys[1] = (int *)w; w += fgnn_align256((size_t)n * sizeof(int));
    int *pay[2];
    pay[0] = pay_out;
    pay[1] = (int *)w; w += fgnn_align256((size_t)n * sizeof(int));
    int *hist = (int *)w; w += fgnn_align256(256 * (size_t)nblocks * sizeof(int));
    int *digit_total = (int *)w; w += fgnn_align256(256 * sizeof(int));
    int *digit_base = (int *)w;
    const int *kin = keys_in;
    const int *pin = pay_in;
    for (int i = 0; i < passes; ++i) {
        int shift = bits * i;
        int *kout = keys[i & 1];
        int *pout = pay[(passes - 1 - i) & 1];      // the last pass lands in pay_out
        hipLaunchKernelGGL(rs_hist_kernel, dim3(nblocks), dim3(RS_TPB), 0, st, kin, n, shift, (1 << bits) - 1, nblocks, hist);
        int rc = fgnn_launch_status("rs_hist_kernel");
        if (rc) return rc;
        hipLaunchKernelGGL(rs_scan_kernel, dim3(1 << bits), dim3(RS_TPB), 0, st, hist, nblocks, digit_total);
        rc = fgnn_launch_status("rs_scan_kernel");
        if (rc) return rc;
        hipLaunchKernelGGL(rs_digit_base_kernel, dim3(1), dim3(256), 0, st, digit_total, 1 << bits, digit_base);
        rc = fgnn_launch_status("rs_digit_base_kernel");
        if (rc) return rc;
        hipLaunchKernelGGL(rs_scatter_kernel, dim3(nblocks), dim3(RS_TPB), 0, st, kin, pin, n, shift, bits, nblocks, hist, digit_base, kout, pout);
        rc = fgnn_launch_status("rs_scatter_kernel");
        if (rc) return rc;
        kin = kout;
        pin = pout;
    }
    *sorted_keys = kin;
    return 0;
}

static int csc_num_hints(int64_t E) { return E > 0 ? (int)((E - 1) >> CSC_HINT_SHIFT) + 2 : 0; }

extern "C" size_t fgnn_csr2csc_workspace_bytes(int n_rows, int n_cols, int64_t E)
{
    (void)n_rows; (void)n_cols;
    return rs_sort_workspace(E) + fgnn_align256((size_t)csc_num_hints(E) * sizeof(int));
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
    const int *sorted = nullptr;
    int rc = rs_sort_pairs(col_ind, nullptr, E, rs_key_bits(n_cols), permute, &sorted, workspace, st);
    if (rc) return rc;
    int *hint = (int *)((char *)workspace + rs_sort_workspace(E));
    const int n_hint = csc_num_hints(E);
    hipLaunchKernelGGL(csc_row_hint_kernel, dim3((unsigned)((n_hint + 255) / 256)), dim3(256), 0, st, E, n_rows, n_hint, row_ptr, hint);
    rc = fgnn_launch_status("csc_row_hint_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(csc_finalize_kernel, dim3((unsigned)((E + 255) / 256)), dim3(256), 0, st, E, n_cols, sorted, permute, row_ptr, hint, col_ptr, row_ind);
    return fgnn_launch_status("csc_finalize_kernel");
}

// ------------------------------------------------------------------------------- COO -> CSR
// Edge list (dst[e], src[e]) -> CSR by destination with sources ascending inside a row, optionally
// merging duplicate edges: what the reference does on the host with scipy's csr_matrix
// (script/train/train_gatconv_our.py:87-91).  Two stable radix sorts (by src, then by dst), a
// first-of-its-group flag, an inclusive scan of the flags, and a compaction.

__global__ __launch_bounds__(256) void gather_i32_kernel(int64_t n, const int *__restrict__ idx, const int *__restrict__ in, int *__restrict__ out)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = in[idx[i]];
}

// flag[q] = 1 when sorted entry q starts a new (dst, src) group (always 1 without dedupe)
__global__ __launch_bounds__(256) void coo_flag_kernel(int64_t n, const int *__restrict__ dsts, const int *__restrict__ srcs, int dedupe, int *__restrict__ flag)
{
    int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (q >= n) return;
    flag[q] = (!dedupe || q == 0 || dsts[q] != dsts[q - 1] || srcs[q] != srcs[q - 1]) ? 1 : 0;
}

#define SC_ITEMS 16
#define SC_TILE (256 * SC_ITEMS)
// Inclusive scan in three steps: per-tile totals, scan of the totals (one workgroup), per-tile scan + offset.
__global__ __launch_bounds__(256) void scan_tile_sums_kernel(int64_t n, const int *__restrict__ in, int *__restrict__ sums)
{
    __shared__ int sh[256];
    int64_t base = (int64_t)blockIdx.x * SC_TILE + (int64_t)threadIdx.x * SC_ITEMS;
    int acc = 0;
#pragma unroll
    for (int k = 0; k < SC_ITEMS; ++k) acc += (base + k < n) ? in[base + k] : 0;
    sh[threadIdx.x] = acc;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) sh[threadIdx.x] += sh[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) sums[blockIdx.x] = sh[0];
}
__global__ __launch_bounds__(256) void scan_sums_kernel(int nt, int *__restrict__ sums, int *__restrict__ total)
{
    __shared__ int sh[256];
    __shared__ int carry;
    if (threadIdx.x == 0) carry = 0;
    __syncthreads();
    for (int base = 0; base < nt; base += 256) {
        int i = base + (int)threadIdx.x;
        int v = i < nt ? sums[i] : 0;
        sh[threadIdx.x] = v;
        __syncthreads();
        for (int off = 1; off < 256; off <<= 1) {
            int t = (int)threadIdx.x >= off ? sh[threadIdx.x - off] : 0;
            __syncthreads();
            sh[threadIdx.x] += t;
            __syncthreads();
        }
        int incl = sh[threadIdx.x];
        int c = carry;
        if (i < nt) sums[i] = c + incl - v;          // exclusive offset of tile i
        __syncthreads();
        if (threadIdx.x == 255) carry = c + incl;
        __syncthreads();
    }
    if (threadIdx.x == 0) *total = carry;
}
__global__ __launch_bounds__(256) void scan_apply_kernel(int64_t n, const int *__restrict__ in, const int *__restrict__ sums, int *__restrict__ out)
{
    __shared__ int sh[256];
    int64_t base = (int64_t)blockIdx.x * SC_TILE + (int64_t)threadIdx.x * SC_ITEMS;
    int v[SC_ITEMS];
    int acc = 0;
#pragma unroll
    for (int k = 0; k < SC_ITEMS; ++k) { v[k] = (base + k < n) ? in[base + k] : 0; acc += v[k]; }
    sh[threadIdx.x] = acc;
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {
        int t = (int)threadIdx.x >= off ? sh[threadIdx.x - off] : 0;
        __syncthreads();
        sh[threadIdx.x] += t;
        __syncthreads();
    }
    int run = sums[blockIdx.x] + sh[threadIdx.x] - acc;
#pragma unroll
    for (int k = 0; k < SC_ITEMS; ++k) {
        run += v[k];
        if (base + k < n) out[base + k] = run;
    }
}

// Library-internal entry points to the sort and the scan (the schedule builder uses them too).
size_t fgnn_rs_sort_workspace(int64_t n) { return rs_sort_workspace(n); }
int fgnn_rs_key_bits(int n_keys) { return rs_key_bits(n_keys); }
int fgnn_rs_sort_pairs(const int *keys_in, const int *pay_in, int64_t n, int key_bits, int *pay_out, const int **sorted_keys, void *workspace,
                       hipStream_t st)
{
    return rs_sort_pairs(keys_in, pay_in, n, key_bits, pay_out, sorted_keys, workspace, st);
}
size_t fgnn_scan_workspace(int64_t n) { return fgnn_align256(((size_t)((n + SC_TILE - 1) / SC_TILE) + 1) * sizeof(int)); }
// out[i] = in[0] + ... + in[i]; *total_dev = the sum of all.  tile_sums: fgnn_scan_workspace(n) bytes.
int fgnn_inclusive_scan_i32(const int *in, int64_t n, int *out, int *tile_sums, int *total_dev, hipStream_t st)
{
    const int nt = (int)((n + SC_TILE - 1) / SC_TILE);
    hipLaunchKernelGGL(scan_tile_sums_kernel, dim3(nt), dim3(256), 0, st, n, in, tile_sums);
    int rc = fgnn_launch_status("scan_tile_sums_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(scan_sums_kernel, dim3(1), dim3(256), 0, st, nt, tile_sums, total_dev);
    rc = fgnn_launch_status("scan_sums_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(scan_apply_kernel, dim3(nt), dim3(256), 0, st, n, in, tile_sums, out);
    return fgnn_launch_status("scan_apply_kernel");
}

// Compaction: the first entry of every group writes its source and destination at the group's
// position; every input edge learns the position of its group.
__global__ __launch_bounds__(256) void coo_compact_kernel(int64_t n, const int *__restrict__ dsts, const int *__restrict__ srcs,
                                                          const int *__restrict__ perm, const int *__restrict__ flag, const int *__restrict__ incl,
                                                          int *__restrict__ col_ind, int *__restrict__ dstc, int *__restrict__ edge_pos)
{
    int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (q >= n) return;
    int pos = incl[q] - 1;
    if (flag[q]) { col_ind[pos] = srcs[q]; dstc[pos] = dsts[q]; }
    if (edge_pos) edge_pos[perm[q]] = pos;
}

// row_ptr from the compacted destinations (ascending); *n_out entries are valid.
__global__ __launch_bounds__(256) void coo_rowptr_kernel(int n_rows, const int *__restrict__ dstc, const int *__restrict__ n_out_dev,
                                                         int *__restrict__ row_ptr, int64_t *__restrict__ n_out)
{
    int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int m = *n_out_dev;
    if (q == 0 && n_out) *n_out = m;
    if (q >= m) return;
    int key = dstc[q];
    int prev = q > 0 ? dstc[q - 1] : -1;
    for (int r = prev + 1; r <= key; ++r) row_ptr[r] = (int)q;
    if (q == m - 1)
        for (int r = key + 1; r <= n_rows; ++r) row_ptr[r] = m;
}

extern "C" size_t fgnn_coo2csr_workspace_bytes(int n_rows, int n_cols, int64_t E)
{
    (void)n_rows; (void)n_cols;
    size_t nt = (size_t)((E + SC_TILE - 1) / SC_TILE);
    // sort scratch | perm1 | keys2 / srcs | perm2 | flag | incl | dstc | tile sums | total
    return rs_sort_workspace(E) + 6 * fgnn_align256((size_t)E * sizeof(int)) + fgnn_align256((nt + 1) * sizeof(int)) + 256;
}

extern "C" int fgnn_coo2csr(int n_rows, int n_cols, int64_t E, const int32_t *dst, const int32_t *src, int dedupe, int32_t *row_ptr,
                            int32_t *col_ind, int64_t *n_out, int32_t *edge_pos, void *workspace, size_t workspace_bytes, void *stream)
{
    FGNN_REQUIRE(n_rows >= 0 && n_cols >= 0 && E >= 0, FGNN_ERR_SHAPE, "fgnn_coo2csr: bad sizes");
    FGNN_REQUIRE(E <= 2147483647LL - RS_TILE, FGNN_ERR_LIMIT, "fgnn_coo2csr: E=%lld exceeds int32 positions", (long long)E);
    FGNN_REQUIRE(row_ptr && n_out && (E == 0 || (dst && src && col_ind)), FGNN_ERR_NULL, "fgnn_coo2csr: NULL argument");
    hipStream_t st = (hipStream_t)stream;
    if (E == 0) {
        hipLaunchKernelGGL(fill_i32_kernel, dim3((unsigned)((n_rows + 1 + 255) / 256)), dim3(256), 0, st, row_ptr, (size_t)n_rows + 1, 0);
        int rc = fgnn_launch_status("fill_i32_kernel");
        if (rc) return rc;
        hipLaunchKernelGGL(fill_i32_kernel, dim3(1), dim3(256), 0, st, (int *)n_out, (size_t)2, 0);    // int64 zero, as a kernel
        return fgnn_launch_status("fill_i32_kernel");
    }
    FGNN_REQUIRE(n_cols >= 1 && n_rows >= 1, FGNN_ERR_SHAPE, "fgnn_coo2csr: edges without rows or columns");
    size_t need = fgnn_coo2csr_workspace_bytes(n_rows, n_cols, E);
    FGNN_REQUIRE(workspace && workspace_bytes >= need, FGNN_ERR_WORKSPACE, "fgnn_coo2csr: workspace %zu < %zu bytes", workspace_bytes, need);
    char *w = (char *)workspace;
    void *sort_ws = w; w += rs_sort_workspace(E);
    size_t eb = fgnn_align256((size_t)E * sizeof(int));
    int *perm1 = (int *)w; w += eb;
    int *tmp = (int *)w; w += eb;          // dst gathered by perm1, later the sorted sources
    int *perm2 = (int *)w; w += eb;
    int *flag = (int *)w; w += eb;
    int *incl = (int *)w; w += eb;
    int *dstc = (int *)w; w += eb;
    const int nt = (int)((E + SC_TILE - 1) / SC_TILE);
    int *sums = (int *)w; w += fgnn_align256(((size_t)nt + 1) * sizeof(int));
    int *total = (int *)w;
    const unsigned ge = (unsigned)((E + 255) / 256);

    const int *sorted = nullptr;
    int rc = rs_sort_pairs(src, nullptr, E, rs_key_bits(n_cols), perm1, &sorted, sort_ws, st);
    if (rc) return rc;
    hipLaunchKernelGGL(gather_i32_kernel, dim3(ge), dim3(256), 0, st, E, perm1, dst, tmp);
    rc = fgnn_launch_status("gather_i32_kernel");
    if (rc) return rc;
    const int *dsts = nullptr;
    rc = rs_sort_pairs(tmp, perm1, E, rs_key_bits(n_rows), perm2, &dsts, sort_ws, st);
    if (rc) return rc;
    hipLaunchKernelGGL(gather_i32_kernel, dim3(ge), dim3(256), 0, st, E, perm2, src, tmp);       // sources in (dst, src) order
    rc = fgnn_launch_status("gather_i32_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(coo_flag_kernel, dim3(ge), dim3(256), 0, st, E, dsts, tmp, dedupe, flag);
    rc = fgnn_launch_status("coo_flag_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(scan_tile_sums_kernel, dim3(nt), dim3(256), 0, st, E, flag, sums);
    rc = fgnn_launch_status("scan_tile_sums_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(scan_sums_kernel, dim3(1), dim3(256), 0, st, nt, sums, total);
    rc = fgnn_launch_status("scan_sums_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(scan_apply_kernel, dim3(nt), dim3(256), 0, st, E, flag, sums, incl);
    rc = fgnn_launch_status("scan_apply_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(coo_compact_kernel, dim3(ge), dim3(256), 0, st, E, dsts, tmp, perm2, flag, incl, col_ind, dstc, edge_pos);
    rc = fgnn_launch_status("coo_compact_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(coo_rowptr_kernel, dim3(ge), dim3(256), 0, st, n_rows, dstc, total, row_ptr, n_out);
    return fgnn_launch_status("coo_rowptr_kernel");
}
