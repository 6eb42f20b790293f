// Row-wise softmax cross-entropy for the training drivers (the loss of script/train/train_gatconv_our.py:166-175,
// torch.nn.CrossEntropyLoss on the logits of all labelled nodes): per row the log-sum-exp and the loss in one pass over the
// logits, and the gradient (softmax - one-hot) * upstream in one more.  Composed from torch operators the same loss is a
// dozen elementwise and reduction kernels over the [N, classes] array (2.4 ms of a 38 ms step at 2.4 M nodes x 47 classes);
// these two passes read it once each.
#include <algorithm>
#include "fgnn_common.h"

// A row is spread over LPR lanes (a power of two <= 64), lane s of its group owns the groups of VEC floats s, s + LPR, ...;
// a wave takes 64 / LPR rows per trip.  Reductions inside a group by xor-shuffles (every lane gets the result).
template <int LPR>
__device__ __forceinline__ float ce_group_max(float v)
{
#pragma unroll
    for (int d = 1; d < LPR; d <<= 1) v = fmaxf(v, __shfl_xor(v, d));
    return v;
}
template <int LPR>
__device__ __forceinline__ float ce_group_sum(float v)
{
#pragma unroll
    for (int d = 1; d < LPR; d <<= 1) v += __shfl_xor(v, d);
    return v;
}

#define CE_MAXG 4       // groups of VEC floats a lane keeps in registers: rows of up to LPR * CE_MAXG * VEC floats

template <int VEC, int LPR>
__global__ __launch_bounds__(256) void ce_forward_kernel(int64_t N, int C, int64_t ld, const float *__restrict__ x, const int64_t *__restrict__ labels,
                                                         float *__restrict__ lse, float *__restrict__ row_loss)
{
    constexpr int RPW = 64 / LPR;
    const int lane = fg_lane(), sub = lane % LPR;
    const int64_t wave = (int64_t)blockIdx.x * 4 + fg_wave(), nwaves = (int64_t)gridDim.x * 4;
    const int G = (C + VEC - 1) / VEC;                           // groups per row (the last one may be partial)
    for (int64_t r0 = wave * RPW; r0 < N; r0 += nwaves * RPW) {
        const int64_t row = r0 + lane / LPR;
        const bool rok = row < N;
        float v[CE_MAXG][VEC];
        float m = -INFINITY;
#pragma unroll
        for (int k = 0; k < CE_MAXG; ++k) {
            const int g = sub + k * LPR;
#pragma unroll
            for (int c = 0; c < VEC; ++c) v[k][c] = -INFINITY;
            if (rok && g < G) {
                const float *p = x + row * ld + (int64_t)g * VEC;
                if constexpr (VEC == 4) {
                    const float4 t = *reinterpret_cast<const float4 *>(p);          // ld % 4 == 0: the whole group lies inside the row's storage
                    v[k][0] = t.x; v[k][1] = t.y; v[k][2] = t.z; v[k][3] = t.w;
#pragma unroll
                    for (int c = 0; c < 4; ++c) if (g * 4 + c >= C) v[k][c] = -INFINITY;   // padding columns
                } else {
                    v[k][0] = p[0];
                }
            }
#pragma unroll
            for (int c = 0; c < VEC; ++c) m = fmaxf(m, v[k][c]);
        }
        m = ce_group_max<LPR>(m);
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < CE_MAXG; ++k)
#pragma unroll
            for (int c = 0; c < VEC; ++c) s += __expf(v[k][c] - m);                  // exp(-inf) = 0
        s = ce_group_sum<LPR>(s);
        if (rok && sub == 0) {
            const int64_t y = labels[row];
            const float l = m + __logf(s);
            lse[row] = l;
            // a label outside [0, C) never indexes the row: its loss is NaN, which no caller can miss
            row_loss[row] = (y < 0 || y >= C) ? __int_as_float(0x7fc00000) : l - x[row * ld + y];
        }
    }
}

// grad[row, c] = (exp(x[row, c] - lse[row]) - [c == label]) * upstream[row]; the padding columns C..ldg-1 of grad get zeros.
template <int VEC, int LPR>
__global__ __launch_bounds__(256) void ce_backward_kernel(int64_t N, int C, int64_t ld, int64_t ldg, const float *__restrict__ x,
                                                          const int64_t *__restrict__ labels, const float *__restrict__ lse,
                                                          const float *__restrict__ upstream, float *__restrict__ grad)
{
    constexpr int RPW = 64 / LPR;
    const int lane = fg_lane(), sub = lane % LPR;
    const int64_t wave = (int64_t)blockIdx.x * 4 + fg_wave(), nwaves = (int64_t)gridDim.x * 4;
    const int GG = (int)((ldg + VEC - 1) / VEC);                 // groups of a gradient row
    for (int64_t r0 = wave * RPW; r0 < N; r0 += nwaves * RPW) {
        const int64_t row = r0 + lane / LPR;
        if (row >= N) continue;
        const float l = lse[row], up = upstream[row];
        const int y = (int)labels[row];
#pragma unroll
        for (int k = 0; k < CE_MAXG; ++k) {
            const int g = sub + k * LPR;
            if (g >= GG) continue;
            float t[VEC];
            if constexpr (VEC == 4) {
                const bool in_x = (int64_t)g * 4 + 4 <= ld;
                const float4 q = in_x ? *reinterpret_cast<const float4 *>(x + row * ld + (int64_t)g * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
                t[0] = q.x; t[1] = q.y; t[2] = q.z; t[3] = q.w;
            } else {
                t[0] = g < C ? x[row * ld + g] : 0.f;
            }
            float o[VEC];
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
                const int col = g * VEC + c;
                o[c] = col < C ? (__expf(t[c] - l) - (col == y ? 1.f : 0.f)) * up : 0.f;
            }
            float *dst = grad + row * ldg + (int64_t)g * VEC;
            if constexpr (VEC == 4) *reinterpret_cast<float4 *>(dst) = make_float4(o[0], o[1], o[2], o[3]);
            else dst[0] = o[0];
        }
    }
}

static inline int ce_pick_lpr(int groups)
{
    int lpr = 1;
    while (lpr < 64 && lpr * CE_MAXG < groups) lpr *= 2;
    return lpr;
}
template <typename Fn>
static inline int ce_dispatch(int vec, int lpr, Fn &&f)
{
#define CE_CASE(L) case L: return vec == 4 ? f.template operator()<4, L>() : f.template operator()<1, L>();
    switch (lpr) { CE_CASE(1) CE_CASE(2) CE_CASE(4) CE_CASE(8) CE_CASE(16) CE_CASE(32) default: return vec == 4 ? f.template operator()<4, 64>() : f.template operator()<1, 64>(); }
#undef CE_CASE
}

extern "C" int fgnn_cross_entropy_forward(int64_t N, int C, int64_t ld, const float *logits, const int64_t *labels, float *lse,
                                          float *row_loss, void *stream)
{
    FGNN_REQUIRE(N >= 0 && C >= 1 && ld >= C, FGNN_ERR_SHAPE, "fgnn_cross_entropy_forward: bad sizes N=%lld C=%d ld=%lld", (long long)N, C, (long long)ld);
    if (N == 0) return 0;
    FGNN_REQUIRE(logits && labels && lse && row_loss, FGNN_ERR_NULL, "fgnn_cross_entropy_forward: NULL argument");
    const int vec = (ld % 4 == 0 && fgnn_aligned16(logits)) ? 4 : 1;
    const int groups = (C + vec - 1) / vec;
    FGNN_REQUIRE(groups <= 64 * CE_MAXG, FGNN_ERR_LIMIT, "fgnn_cross_entropy_forward: %d classes unsupported (at most %d, or %d with rows that are multiples of four floats)",
                 C, 64 * CE_MAXG, 256 * CE_MAXG);
    const int lpr = ce_pick_lpr(groups);
    const int64_t rows_per_block = 4 * (64 / lpr);
    const unsigned grid = (unsigned)std::min<int64_t>((N + rows_per_block - 1) / rows_per_block, 16384);
    return ce_dispatch(vec, lpr, [&]<int VEC, int LPR>() -> int {
        hipLaunchKernelGGL((ce_forward_kernel<VEC, LPR>), dim3(grid), dim3(256), 0, (hipStream_t)stream, N, C, ld, logits, labels, lse, row_loss);
        return fgnn_launch_status("ce_forward_kernel");
    });
}

extern "C" int fgnn_cross_entropy_backward(int64_t N, int C, int64_t ld, int64_t ld_grad, const float *logits, const int64_t *labels,
                                           const float *lse, const float *upstream, float *grad_logits, void *stream)
{
    FGNN_REQUIRE(N >= 0 && C >= 1 && ld >= C && ld_grad >= C, FGNN_ERR_SHAPE, "fgnn_cross_entropy_backward: bad sizes N=%lld C=%d ld=%lld ld_grad=%lld",
                 (long long)N, C, (long long)ld, (long long)ld_grad);
    if (N == 0) return 0;
    FGNN_REQUIRE(logits && labels && lse && upstream && grad_logits, FGNN_ERR_NULL, "fgnn_cross_entropy_backward: NULL argument");
    const int vec = (ld % 4 == 0 && ld_grad % 4 == 0 && fgnn_aligned16(logits) && fgnn_aligned16(grad_logits)) ? 4 : 1;
    const int groups = (int)((ld_grad + vec - 1) / vec);
    FGNN_REQUIRE(groups <= 64 * CE_MAXG, FGNN_ERR_LIMIT, "fgnn_cross_entropy_backward: rows of %lld floats unsupported", (long long)ld_grad);
    const int lpr = ce_pick_lpr(groups);
    const int64_t rows_per_block = 4 * (64 / lpr);
    const unsigned grid = (unsigned)std::min<int64_t>((N + rows_per_block - 1) / rows_per_block, 16384);
    return ce_dispatch(vec, lpr, [&]<int VEC, int LPR>() -> int {
        hipLaunchKernelGGL((ce_backward_kernel<VEC, LPR>), dim3(grid), dim3(256), 0, (hipStream_t)stream, N, C, ld, ld_grad, logits, labels, lse,
                           upstream, grad_logits);
        return fgnn_launch_status("ce_backward_kernel");
    });
}
