// Fused GAT forward / backward for gfx950.
//
// Forward (one gather pass over CSR rows): per work item (a row, or a segment of a long row) a
// wave streams over the edges 8 at a time.  The 64 lanes own the floats of a feature row (one
// 128-bit load per lane and edge); every lane also reads attn_col[j, head of its floats] and
// computes the softmax numerator itself, with an online (running-maximum) softmax, so there is
// no separate maximum pass, no cross-lane traffic and no LDS.  Next to the plain sum T the wave
// keeps P, the sum over edges with a positive pre-activation; T and P give both
//   out  = T / s                         and
//   out2 = (slope*T + (1-slope)*P) / s   = sum_p alpha_p * lrelu'(e_p) * in_feat[j_p],
// which turns the gradient of attn_row into node-wise dot products in the backward.
//
// Backward (one gather pass over CSC columns): a node-wise pre-kernel forms
//   delta[i,h] = <g[i,h,:], out[i,h,:]>,  grad_attn_row[i,h] = <g[i,h,:], out2[i,h,:]> - delta*c[i,h]
// and packs (attn_row, max, 1/sum, delta) per (node, head).  The column pass recomputes alpha
// from that record, accumulates T = sum alpha*g[i] (= grad_feat) and P likewise, and finishes with
//   grad_attn_col[j,h] = <in_feat[j,h,:], slope*T + (1-slope)*P> - sum_i alpha*lrelu'(e)*delta[i,h].
// No atomics anywhere: results are bit-reproducible.
//
// Math contract: src/fused_gat/fused_gat_SM.cu:193-286 (forward), :560-607, :656-732, :734-801
// (backward) of the reference; LeakyReLU derivative at 0 is `slope` as in torch.
#include <algorithm>
#include "fgnn_common.h"

struct GatFwdP {
    const fgnn_item *items; int n_items;
    const int *ptr; const int *idx;
    const float *ar; const float *ac; const float *x;
    float *out; float *emax; float *esum; float *out2; float *cc;
    float *part;
    int N, H, F, HF; float slope;
    int hp_shift;   // pair layout of the batches (gat_fwd_pair_batch): lane = (edge of the batch << hp_shift) | head
};

// Partial layout (floats): T[HF] | P[HF] (AUX only) | m[H] | s[H] | cp[H]
__host__ __device__ static inline int gat_fwd_pw(int HF, int H, bool aux) { return ((aux ? 2 : 1) * HF + 3 * H + 3) & ~3; }

// One batch of UB edges of the forward: UB feature rows and UB x R attention scores are fetched
// together (every lane reads the score of the head its features belong to), then the running
// maximum of the online softmax is raised once for the batch and the rows are accumulated.
// Scores are kept in log2 units (LeakyReLU commutes with the positive factor log2(e)), so the
// numerator is one v_exp_f32.  TAIL: the batch may reach past the end of the chunk.
template <int VEC, int R, bool AUX, bool FULL, int UB, bool TAIL, bool SLE1>
__device__ __forceinline__ void gat_fwd_batch(const GatFwdP &p, const fg_lanemap<VEC, R> &lm, const uint32_t (&boff)[R],
                                              const uint32_t (&hoff)[R], int idv, int t, int cnt, const float (&arh)[R],
                                              float (&m)[R], float (&s)[R], float (&cp)[R], fg_vec<VEC> (&T)[R], fg_vec<VEC> (&P)[R])
{
    fg_vec<VEC> ld[UB][R];
    float ev[UB][R];
    const size_t row_bytes = (size_t)p.HF * sizeof(float), sc_bytes = (size_t)p.H * sizeof(float);
#pragma unroll
    for (int u = 0; u < UB; ++u) {
        size_t j = (size_t)(unsigned)__builtin_amdgcn_readlane(idv, t + u);
        const char *base = (const char *)p.x + j * row_bytes;
        const char *acb = (const char *)p.ac + j * sc_bytes;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (FULL || lm.ok[r]) { ld[u][r].load_off(base, boff[r]); ev[u][r] = *(const float *)(acb + hoff[r]); }
            else { ld[u][r].zero(); ev[u][r] = 0.f; }
        }
    }
    float bm[R];
#pragma unroll
    for (int r = 0; r < R; ++r) bm[r] = -INFINITY;
#pragma unroll
    for (int u = 0; u < UB; ++u) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float v = fg_lrelu_t<SLE1>(fmaf(ev[u][r], FGNN_LOG2E, arh[r]), p.slope);
            if (TAIL) v = ((t + u) < cnt) ? v : -INFINITY;      // wave-uniform: edges past the chunk get weight 0
            ev[u][r] = v;
            bm[r] = fmaxf(bm[r], v);
        }
    }
    bool raised = false;
#pragma unroll
    for (int r = 0; r < R; ++r) raised |= bm[r] > m[r];
    if (__builtin_amdgcn_ballot_w64(raised) != 0ull) {          // the running maximum rarely moves after the first batches
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float mn = fmaxf(m[r], bm[r]);
            float sc = __builtin_amdgcn_exp2f(m[r] - mn);        // 1 when this head's maximum did not move, 0 on the first batch
            m[r] = mn;
            T[r].scale(sc);
            s[r] *= sc;
            if (AUX) { P[r].scale(sc); cp[r] *= sc; }
        }
    }
#pragma unroll
    for (int u = 0; u < UB; ++u) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float w = __builtin_amdgcn_exp2f(ev[u][r] - m[r]);
            T[r].fma(w, ld[u][r]);
            s[r] += w;
            if (AUX) {
                float wp = ev[u][r] > 0.f ? w : 0.f;
                P[r].fma(wp, ld[u][r]);
                cp[r] += wp;
            }
        }
    }
}

// The same batch with the scores handled in a PAIR layout: lane (u << hp_shift) | h owns (edge u of the
// batch, head h).  It alone reads attn_col of that pair and does the LeakyReLU / exp2 / running-maximum
// arithmetic, once per batch instead of once per edge on every lane; the feature lanes fetch the weight
// of (their edge, their head) with ds_bpermute.  The online-softmax state lives in the pair layout: m is
// the head's running maximum (equal in all edge slots of a head), s and cp are per-slot partial sums.
struct GatFwdPair { int u, h; bool ok; float arh, m, s, cp; };
// attn_col of the lane's pair in the batch that starts at entry t of the chunk (0 for a slot without an
// edge).  Issued one batch ahead of its use, so that the feature-row loads never wait behind it.
__device__ __forceinline__ float gat_fwd_pair_fetch(const GatFwdP &p, const GatFwdPair &pr, int idv, int t, int cnt)
{
    const int jp = __builtin_amdgcn_ds_bpermute(((t + pr.u) & 63) << 2, idv);      // (lane exchanges stay outside divergent code)
    float acv = 0.f;
    if (pr.ok && t + pr.u < cnt) acv = p.ac[(size_t)(unsigned)jp * p.H + pr.h];
    return acv;
}
template <int VEC, int R, bool AUX, bool FULL, int UB, bool SLE1>
__device__ __forceinline__ void gat_fwd_pair_batch(const GatFwdP &p, const fg_lanemap<VEC, R> &lm, const uint32_t (&boff)[R],
                                                   int idv, int t, int cnt, int lane, GatFwdPair &pr, float &acv,
                                                   fg_vec<VEC> (&T)[R], fg_vec<VEC> (&P)[R])
{
    float acn = 0.f;
    if (t + UB < cnt) acn = gat_fwd_pair_fetch(p, pr, idv, t + UB, cnt);        // wave-uniform
    fg_vec<VEC> ld[UB][R];
    const uint32_t row_bytes = (uint32_t)p.HF * 4u;
    uint32_t bo[R];
#pragma unroll
    for (int r = 0; r < R; ++r) bo[r] = fg_pin(boff[r]);
#pragma unroll
    for (int u = 0; u < UB; ++u) {
        uint64_t j = (uint64_t)(uint32_t)__builtin_amdgcn_readlane(idv, (t + u) & 63);      // past the chunk: any valid row, weight 0
        fg_gptr base = fg_uniform_ptr((const char *)p.x + j * row_bytes);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (FULL || lm.ok[r]) ld[u][r].load_off(base, bo[r]); else ld[u][r].zero();
        }
    }
    const bool live = pr.ok && t + pr.u < cnt;
    const float v = live ? fg_lrelu_t<SLE1>(fmaf(acv, FGNN_LOG2E, pr.arh), p.slope) : -INFINITY;
    float bm = v;                                                   // the head's maximum over the batch
    for (int sft = 1 << p.hp_shift; sft < 64; sft <<= 1) bm = fmaxf(bm, fg_bperm(bm, lane ^ sft));
    if (__builtin_amdgcn_ballot_w64(bm > pr.m) != 0ull) {           // the running maximum rarely moves after the first batches
        const float mn = fmaxf(pr.m, bm);
        const float sc = __builtin_amdgcn_exp2f(pr.m - mn);         // 1 when this head's maximum did not move, 0 on the first batch
        pr.m = mn; pr.s *= sc; pr.cp *= sc;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float scf = fg_bperm(sc, lm.hd[r]);
            T[r].scale(scf);
            if (AUX) P[r].scale(scf);
        }
    }
    const float w = __builtin_amdgcn_exp2f(v - pr.m);               // 0 for the slots without an edge
    const float wp = v > 0.f ? w : 0.f;
    pr.s += w; pr.cp += wp;
    // w >= 0, so one exchange carries both weights: the sign says whether the pre-activation was positive
    const float ws = (!AUX || v > 0.f) ? w : -w;
#pragma unroll
    for (int u = 0; u < UB; ++u) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int src = ((u << p.hp_shift) + lm.hd[r]) << 2;
            const float a = __int_as_float(__builtin_amdgcn_ds_bpermute(src, __float_as_int(ws)));
            T[r].fma(AUX ? fabsf(a) : a, ld[u][r]);
            if (AUX) P[r].fma(fg_relu_bits(a), ld[u][r]);
        }
    }
    acv = acn;
}

template <int VEC, int R, bool AUX, bool FULL, bool SLE1, bool PAIR>
__global__ __launch_bounds__(FGNN_TPB) void gat_fwd_kernel(GatFwdP p)
{
    int row, b, e, slot;
    if (!fg_get_item(p.items, p.n_items, p.ptr, row, b, e, slot)) return;
    const int lane = fg_lane();
    const int H = p.H;
    fg_lanemap<VEC, R> lm;
    lm.init(lane, p.HF, p.F);
    const float slope = p.slope;

    fg_vec<VEC> T[R], P[R];
    float arh[R], m[R], s[R], cp[R];
    uint32_t boff[R], hoff[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        T[r].zero(); P[r].zero(); s[r] = 0.f; cp[r] = 0.f; m[r] = -INFINITY;
        arh[r] = p.ar[(size_t)row * H + lm.hd[r]] * FGNN_LOG2E;
        boff[r] = (uint32_t)lm.eoff[r] * 4u;
        hoff[r] = (uint32_t)lm.hd[r] * 4u;
    }
    // Feature rows in flight per wave: eight where the rows are long and mostly hit L2 (the pair layout's case), four on
    // graphs of short rows out of HBM, where the registers saved buy an eighth wave per SIMD (2.4 M nodes x 26 entries,
    // 8 x 32: backward 11.6 -> 10.9 ms; the 492-entry rows of the 115 M-edge graph lose 2-3 % with four).
    constexpr int U = (R >= 8) ? 1 : (PAIR || R > 2 ? 8 : 4) / R;
    GatFwdPair pr;
    pr.u = lane >> p.hp_shift; pr.h = lane & ((1 << p.hp_shift) - 1);
    pr.ok = PAIR && pr.h < H && pr.u < U;
    pr.arh = pr.ok ? p.ar[(size_t)row * H + pr.h] * FGNN_LOG2E : 0.f;
    pr.m = pr.ok ? -INFINITY : 0.f; pr.s = 0.f; pr.cp = 0.f;
    for (int c = b; c < e; c += 64) {
        int q = c + lane;
        int cnt = min(64, e - c);
        int idv = p.idx[q < e ? q : c];            // lanes past the end repeat a valid id
        int t = 0;
        if constexpr (PAIR) {
            float acv = gat_fwd_pair_fetch(p, pr, idv, 0, cnt);
            for (; t + U <= cnt; t += U) gat_fwd_pair_batch<VEC, R, AUX, FULL, U, SLE1>(p, lm, boff, idv, t, cnt, lane, pr, acv, T, P);
            if constexpr (U >= 4) {
                if (cnt - t > U / 2) gat_fwd_pair_batch<VEC, R, AUX, FULL, U, SLE1>(p, lm, boff, idv, t, cnt, lane, pr, acv, T, P);
                else if (cnt - t > 0) gat_fwd_pair_batch<VEC, R, AUX, FULL, U / 2, SLE1>(p, lm, boff, idv, t, cnt, lane, pr, acv, T, P);
            } else {
                if (cnt - t > 0) gat_fwd_pair_batch<VEC, R, AUX, FULL, U, SLE1>(p, lm, boff, idv, t, cnt, lane, pr, acv, T, P);
            }
        } else {
            for (; t + U <= cnt; t += U) gat_fwd_batch<VEC, R, AUX, FULL, U, false, SLE1>(p, lm, boff, hoff, idv, t, cnt, arh, m, s, cp, T, P);
            if constexpr (U >= 4) {
                if (cnt - t > U / 2) gat_fwd_batch<VEC, R, AUX, FULL, U, true, SLE1>(p, lm, boff, hoff, idv, t, cnt, arh, m, s, cp, T, P);
                else if (cnt - t > 0) gat_fwd_batch<VEC, R, AUX, FULL, U / 2, true, SLE1>(p, lm, boff, hoff, idv, t, cnt, arh, m, s, cp, T, P);
            } else {
                if (cnt - t > 0) gat_fwd_batch<VEC, R, AUX, FULL, U, true, SLE1>(p, lm, boff, hoff, idv, t, cnt, arh, m, s, cp, T, P);
            }
        }
    }
    if constexpr (PAIR) {
        // back to the feature layout: per head the maximum and the sums over the edge slots
        float st = pr.s, ct = pr.cp;
        for (int sft = 1 << p.hp_shift; sft < 64; sft <<= 1) { st += fg_bperm(st, lane ^ sft); ct += fg_bperm(ct, lane ^ sft); }
#pragma unroll
        for (int r = 0; r < R; ++r) { m[r] = fg_bperm(pr.m, lm.hd[r]); s[r] = fg_bperm(st, lm.hd[r]); cp[r] = fg_bperm(ct, lm.hd[r]); }
    }

    // The maximum leaves the kernel in natural units.  Its rounding is absorbed into the sums, so
    // that (max, sum) stay an exact pair for whoever rebuilds alpha = exp(e - max) / sum from them
    // with max * log2(e) as the exponent offset (the backward does).
    float mnat[R], fix[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        mnat[r] = m[r] * FGNN_LN2;
        fix[r] = (b < e) ? __builtin_amdgcn_exp2f(m[r] - mnat[r] * FGNN_LOG2E) : 1.f;
    }
    if (slot < 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (!(FULL || lm.ok[r])) continue;
            float inv = s[r] > 0.f ? 1.f / s[r] : 0.f;
            size_t o = (size_t)row * p.HF + lm.eoff[r];
            if (AUX) {
                fg_vec<VEC> o2 = T[r].lin(slope * inv, (1.f - slope) * inv, P[r]);
                o2.store_nt(p.out2 + o);
            }
            T[r].scale(inv);
            T[r].store_nt(p.out + o);
            if (lm.eoff[r] % p.F == 0) {
                size_t so = (size_t)row * H + lm.hd[r];
                p.emax[so] = (b < e) ? mnat[r] : -1e38f;
                p.esum[so] = s[r] * fix[r];
                if (AUX) p.cc[so] = (cp[r] + slope * (s[r] - cp[r])) * inv;
            }
        }
    } else {
        float *pp = p.part + (size_t)slot * gat_fwd_pw(p.HF, H, AUX);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (!(FULL || lm.ok[r])) continue;
            T[r].scale(fix[r]);
            T[r].store_nt(pp + lm.eoff[r]);
            if (AUX) { P[r].scale(fix[r]); P[r].store_nt(pp + p.HF + lm.eoff[r]); }
            if (lm.eoff[r] % p.F == 0) {
                float *st = pp + (AUX ? 2 : 1) * p.HF;
                st[lm.hd[r]] = mnat[r];
                st[H + lm.hd[r]] = s[r] * fix[r];
                st[2 * H + lm.hd[r]] = cp[r] * fix[r];
            }
        }
    }
}

// The forward for rows narrower than a wave (H*F <= 128 floats, 16-byte aligned): the wave is
// cut into G lane groups (fg_packmap) that take different edges of the row with the same load
// instruction, each with its own online softmax state; the groups are combined by a log-sum-exp
// butterfly before the row is written.
// PAIR: the scores are handled in the pair layout of gat_fwd_pair_batch, one lane per (entry of the
// batch of 8*G, head); the wave then keeps ONE running maximum per head, so the groups' accumulators
// are plain partial sums.
// n_head: the items this form takes (all of them, or the head of a list whose short items go to gat_fwd_rowpack_items).
template <int G, bool AUX, bool SLE1, bool PAIR, int U = 8>
__device__ __forceinline__ void gat_fwd_packed_item(const GatFwdP &p, int n_head)
{
    int row, b, e, slot;
    if (!fg_get_item(p.items, n_head, p.ptr, row, b, e, slot)) return;
    const int lane = fg_lane();
    const int H = p.H;
    fg_packmap<G> pm;
    pm.init(lane, p.HF, p.F);
    const float slope = p.slope;
    fg_vec<4> T, P;
    T.zero(); P.zero();
    float s = 0.f, cp = 0.f, m = -INFINITY;
    const float arh = p.ar[(size_t)row * H + pm.hd] * FGNN_LOG2E;
    // U: load instructions in flight
    GatFwdPair pr;
    pr.u = lane >> p.hp_shift; pr.h = lane & ((1 << p.hp_shift) - 1);
    pr.ok = PAIR && pr.h < H && pr.u < U * G;
    pr.arh = pr.ok ? p.ar[(size_t)row * H + pr.h] * FGNN_LOG2E : 0.f;
    pr.m = pr.ok ? -INFINITY : 0.f; pr.s = 0.f; pr.cp = 0.f;
    for (int c = b; c < e; c += 64) {
        int q = c + lane;
        int cnt = min(64, e - c);
        int idv = p.idx[q < e ? q : c];
        float acv = 0.f;
        if constexpr (PAIR) acv = gat_fwd_pair_fetch(p, pr, idv, 0, cnt);
        for (int t = 0; t < cnt; t += U * G) {
            fg_vec<4> ld[U];
            float ev[U];
            if constexpr (PAIR) {
                float acn = 0.f;
                if (t + U * G < cnt) acn = gat_fwd_pair_fetch(p, pr, idv, t + U * G, cnt);      // wave-uniform
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int ei = t + u * G + pm.grp;
                    const size_t j = (size_t)(unsigned)__builtin_amdgcn_ds_bpermute((ei & 63) << 2, idv);
                    if (ei < cnt && pm.ok) ld[u].load(p.x + j * p.HF + pm.eoff); else ld[u].zero();
                }
                const bool live = pr.ok && t + pr.u < cnt;
                const float v = live ? fg_lrelu_t<SLE1>(fmaf(acv, FGNN_LOG2E, pr.arh), slope) : -INFINITY;
                float bm = v;
                for (int sft = 1 << p.hp_shift; sft < 64; sft <<= 1) bm = fmaxf(bm, fg_bperm(bm, lane ^ sft));
                if (__builtin_amdgcn_ballot_w64(bm > pr.m) != 0ull) {
                    const float mn = fmaxf(pr.m, bm);
                    const float sc = __builtin_amdgcn_exp2f(pr.m - mn);
                    pr.m = mn; pr.s *= sc; pr.cp *= sc;
                    const float scf = fg_bperm(sc, pm.hd);
                    T.scale(scf);
                    if (AUX) P.scale(scf);
                }
                const float w = __builtin_amdgcn_exp2f(v - pr.m);       // 0 for the slots without an edge
                const float wp = v > 0.f ? w : 0.f;
                pr.s += w; pr.cp += wp;
                const float ws = (!AUX || v > 0.f) ? w : -w;            // the sign carries "pre-activation positive"
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int src = (((u * G + pm.grp) << p.hp_shift) + pm.hd) << 2;
                    const float a = __int_as_float(__builtin_amdgcn_ds_bpermute(src, __float_as_int(ws)));
                    T.fma(AUX ? fabsf(a) : a, ld[u]);
                    if (AUX) P.fma(fg_relu_bits(a), ld[u]);
                }
                acv = acn;
                continue;
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ei = t + u * G + pm.grp;
                const size_t j = (size_t)(unsigned)__builtin_amdgcn_ds_bpermute((ei & 63) << 2, idv);
                if (ei < cnt && pm.ok) { ld[u].load(p.x + j * p.HF + pm.eoff); ev[u] = p.ac[j * H + pm.hd]; }
                else { ld[u].zero(); ev[u] = 0.f; }
            }
            float bm = -INFINITY;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float v = fg_lrelu_t<SLE1>(fmaf(ev[u], FGNN_LOG2E, arh), slope);
                v = ((t + u * G + pm.grp) < cnt && pm.ok) ? v : -INFINITY;      // no edge for this lane: weight 0
                ev[u] = v;
                bm = fmaxf(bm, v);
            }
            if (__builtin_amdgcn_ballot_w64(bm > m) != 0ull) {
                float mn = fmaxf(m, bm);
                float sc = (mn == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m - mn);
                m = mn;
                T.scale(sc);
                s *= sc;
                if (AUX) { P.scale(sc); cp *= sc; }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float w = (ev[u] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(ev[u] - m);
                T.fma(w, ld[u]);
                s += w;
                if (AUX) {
                    float wp = ev[u] > 0.f ? w : 0.f;
                    P.fma(wp, ld[u]);
                    cp += wp;
                }
            }
        }
    }
    if constexpr (PAIR) {
        // one maximum per head for the whole wave: the groups add up; sums over the entry slots
        fg_pack_reduce<G>(T, lane);
        if (AUX) fg_pack_reduce<G>(P, lane);
        float st = pr.s, ct = pr.cp;
        for (int sft = 1 << p.hp_shift; sft < 64; sft <<= 1) { st += fg_bperm(st, lane ^ sft); ct += fg_bperm(ct, lane ^ sft); }
        m = fg_bperm(pr.m, pm.hd); s = fg_bperm(st, pm.hd); cp = fg_bperm(ct, pm.hd);
    }
    // combine the lane groups: (m, s, cp, T, P) of the partner group, rescaled to the common maximum
#pragma unroll
    for (int step = PAIR ? 64 : 64 / G; step < 64; step <<= 1) {
        const int o = lane ^ step;
        float mo = fg_bperm(m, o);
        float mn = fmaxf(m, mo);
        float a = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - mn);
        float bb = (mo == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mo - mn);
        fg_vec<4> To;
        To.v = make_float4(fg_bperm(T.v.x, o), fg_bperm(T.v.y, o), fg_bperm(T.v.z, o), fg_bperm(T.v.w, o));
        T = T.lin(a, bb, To);
        s = a * s + bb * fg_bperm(s, o);
        if (AUX) {
            fg_vec<4> Po;
            Po.v = make_float4(fg_bperm(P.v.x, o), fg_bperm(P.v.y, o), fg_bperm(P.v.z, o), fg_bperm(P.v.w, o));
            P = P.lin(a, bb, Po);
            cp = a * cp + bb * fg_bperm(cp, o);
        }
        m = mn;
    }
    if (!(pm.ok && pm.grp == 0)) return;
    // same epilogue as gat_fwd_kernel: the maximum leaves in natural units, its rounding goes into the sums
    const float mnat = m * FGNN_LN2;
    const float fix = (b < e) ? __builtin_amdgcn_exp2f(m - mnat * FGNN_LOG2E) : 1.f;
    if (slot < 0) {
        float inv = s > 0.f ? 1.f / s : 0.f;
        size_t o = (size_t)row * p.HF + pm.eoff;
        if (AUX) {
            fg_vec<4> o2 = T.lin(slope * inv, (1.f - slope) * inv, P);
            o2.store_nt(p.out2 + o);
        }
        T.scale(inv);
        T.store_nt(p.out + o);
        if (pm.eoff % p.F == 0) {
            size_t so = (size_t)row * H + pm.hd;
            p.emax[so] = (b < e) ? mnat : -1e38f;
            p.esum[so] = s * fix;
            if (AUX) p.cc[so] = (cp + slope * (s - cp)) * inv;
        }
    } else {
        float *pp = p.part + (size_t)slot * gat_fwd_pw(p.HF, H, AUX);
        T.scale(fix);
        T.store_nt(pp + pm.eoff);
        if (AUX) { P.scale(fix); P.store_nt(pp + p.HF + pm.eoff); }
        if (pm.eoff % p.F == 0) {
            float *st = pp + (AUX ? 2 : 1) * p.HF;
            st[pm.hd] = mnat;
            st[H + pm.hd] = s * fix;
            st[2 * H + pm.hd] = cp * fix;
        }
    }
}

// The packed forward with the lane groups on DIFFERENT items: group g of a wave takes a work item of its own and walks it
// alone (its LPR lanes fetch LPR ids at a time, four gathered rows of the group in flight: eight cost a wave per SIMD in
// registers and 4 % in time), so one load instruction fetches a row for each of G destinations and nothing is combined at
// the end.  Per-lane scores (no pair layout).
template <int G, bool AUX, bool SLE1>
__device__ __forceinline__ void gat_fwd_rowpack_items(const GatFwdP &p, int bucketed, int first, int w)
{
    constexpr int LPR = 64 / G, U = 4;
    const int lane = fg_lane();
    const int H = p.H;
    fg_packmap<G> pm;
    pm.init(lane, p.HF, p.F);
    const int sl = lane & (LPR - 1), gbase = lane - sl;
    const int it = fg_group_slot(G, pm.grp, bucketed, first, w);
    int row = -1, b = 0, e = 0, slot = -1;
    if (it < p.n_items) {
        if (p.items) { const fgnn_item q = p.items[it]; row = q.row; b = q.begin; e = q.end; slot = q.slot; }
        else { row = it; b = p.ptr[it]; e = p.ptr[it + 1]; }
    }
    if (row < 0) { b = 0; e = 0; }                                    // padding item or past the list: nothing to walk or store
    if (__builtin_amdgcn_ballot_w64(row >= 0) == 0ull) return;
    const float slope = p.slope;
    fg_vec<4> T, P;
    T.zero(); P.zero();
    float s = 0.f, cp = 0.f, m = -INFINITY;
    const float arh = row >= 0 ? p.ar[(size_t)row * H + pm.hd] * FGNN_LOG2E : 0.f;
    for (int c = b; __builtin_amdgcn_ballot_w64(c < e) != 0ull; c += LPR) {
        const int cnt = min(LPR, e - c);                              // <= 0: this group is done
        int idv = 0;
        if (c < e) idv = p.idx[c + sl < e ? c + sl : c];              // idle lanes repeat a valid id
        for (int t = 0; __builtin_amdgcn_ballot_w64(t < cnt) != 0ull; t += U) {
            fg_vec<4> ld[U];
            float ev[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ei = t + u;
                const size_t j = (size_t)(unsigned)__builtin_amdgcn_ds_bpermute((gbase + (ei & (LPR - 1))) << 2, idv);
                if (ei < cnt && pm.ok) { ld[u].load(p.x + j * p.HF + pm.eoff); ev[u] = p.ac[j * H + pm.hd]; }
                else { ld[u].zero(); ev[u] = 0.f; }
            }
            float bm = -INFINITY;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float v = fg_lrelu_t<SLE1>(fmaf(ev[u], FGNN_LOG2E, arh), slope);
                v = (t + u < cnt && pm.ok) ? v : -INFINITY;           // no edge for this lane: weight 0
                ev[u] = v;
                bm = fmaxf(bm, v);
            }
            if (__builtin_amdgcn_ballot_w64(bm > m) != 0ull) {
                const float mn = fmaxf(m, bm);
                const float sc = (mn == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m - mn);
                m = mn;
                T.scale(sc);
                s *= sc;
                if (AUX) { P.scale(sc); cp *= sc; }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const float w = (ev[u] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(ev[u] - m);
                T.fma(w, ld[u]);
                s += w;
                if (AUX) {
                    const float wp = ev[u] > 0.f ? w : 0.f;
                    P.fma(wp, ld[u]);
                    cp += wp;
                }
            }
        }
    }
    if (!pm.ok || row < 0) return;
    // same epilogue as gat_fwd_kernel: the maximum leaves in natural units, its rounding goes into the sums
    const float mnat = m * FGNN_LN2;
    const float fix = (b < e) ? __builtin_amdgcn_exp2f(m - mnat * FGNN_LOG2E) : 1.f;
    if (slot < 0) {
        const float inv = s > 0.f ? 1.f / s : 0.f;
        const size_t o = (size_t)row * p.HF + pm.eoff;
        if (AUX) {
            fg_vec<4> o2 = T.lin(slope * inv, (1.f - slope) * inv, P);
            o2.store_nt(p.out2 + o);
        }
        T.scale(inv);
        T.store_nt(p.out + o);
        if (pm.eoff % p.F == 0) {
            const size_t so = (size_t)row * H + pm.hd;
            p.emax[so] = (b < e) ? mnat : -1e38f;
            p.esum[so] = s * fix;
            if (AUX) p.cc[so] = (cp + slope * (s - cp)) * inv;
        }
    } else {
        float *pp = p.part + (size_t)slot * gat_fwd_pw(p.HF, H, AUX);
        T.scale(fix);
        T.store_nt(pp + pm.eoff);
        if (AUX) { P.scale(fix); P.store_nt(pp + p.HF + pm.eoff); }
        if (pm.eoff % p.F == 0) {
            float *st = pp + (AUX ? 2 : 1) * p.HF;
            st[pm.hd] = mnat;
            st[H + pm.hd] = s * fix;
            st[2 * H + pm.hd] = cp * fix;
        }
    }
}

template <int G, bool AUX, bool SLE1, bool PAIR>
__global__ __launch_bounds__(FGNN_TPB) void gat_fwd_packed_kernel(GatFwdP p)
{
    gat_fwd_packed_item<G, AUX, SLE1, PAIR>(p, p.n_items);
}
// One launch for a list with a long head: the first head_blocks workgroups put a wave on each of the `first` leading items,
// the others give every lane group an item of the rest.  The head is launched first, so its long items run while the short
// ones fill the rest of the machine (as two launches the second would wait for the longest item of the first).
template <int G, bool AUX, bool SLE1, bool PAIR>
__global__ __launch_bounds__(FGNN_TPB) void gat_fwd_mixed_kernel(GatFwdP p, int bucketed, int first, unsigned head_blocks)
{
    if (blockIdx.x < head_blocks) gat_fwd_packed_item<G, AUX, SLE1, PAIR, 4>(p, first);
    else gat_fwd_rowpack_items<G, AUX, SLE1>(p, bucketed, first, (int)(blockIdx.x - head_blocks));
}

// Merge of the segments of split rows: log-sum-exp combination of (m, s, T, P).
template <int VEC, int R, bool AUX>
__global__ __launch_bounds__(FGNN_TPB) void gat_fwd_merge_kernel(GatFwdP p, const fgnn_split *split, int n_split)
{
    int w = fg_uni((int)blockIdx.x * FGNN_WPB + fg_wave());
    if (w >= n_split) return;
    fgnn_split sp = split[w];
    const int row = fg_uni(sp.row), first = fg_uni(sp.first_slot), nseg = fg_uni(sp.nseg);
    const int lane = fg_lane();
    const int H = p.H, HF = p.HF;
    const int pw = gat_fwd_pw(HF, H, AUX);
    const float slope = p.slope;
    fg_lanemap<VEC, R> lm;
    lm.init(lane, HF, p.F);
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (!lm.ok[r]) continue;
        const int h = lm.hd[r];
        const float *base = p.part + (size_t)first * pw;
        const int so = (AUX ? 2 : 1) * HF;
        float M = -INFINITY;
        for (int g = 0; g < nseg; ++g) M = fmaxf(M, base[(size_t)g * pw + so + h]);
        fg_vec<VEC> T, P;
        T.zero(); P.zero();
        float s = 0.f, cp = 0.f;
        for (int g = 0; g < nseg; ++g) {
            const float *pg = base + (size_t)g * pw;
            float sc = __expf(pg[so + h] - M);
            fg_vec<VEC> t; t.load(pg + lm.eoff[r]);
            T.fma(sc, t);
            if (AUX) { fg_vec<VEC> q; q.load(pg + HF + lm.eoff[r]); P.fma(sc, q); }
            s += sc * pg[so + H + h];
            cp += sc * pg[so + 2 * H + h];
        }
        float inv = s > 0.f ? 1.f / s : 0.f;
        size_t o = (size_t)row * HF + lm.eoff[r];
        if (AUX) { fg_vec<VEC> o2 = T.lin(slope * inv, (1.f - slope) * inv, P); o2.store(p.out2 + o); }
        T.scale(inv);
        T.store(p.out + o);
        if (lm.eoff[r] % p.F == 0) {
            size_t q = (size_t)row * H + h;
            p.emax[q] = M; p.esum[q] = s;
            if (AUX) p.cc[q] = (cp + slope * (s - cp)) * inv;
        }
    }
}

// Per-edge stash of the stash variants: e_lrelu[p,h] and e_softmax[p,h] from the saved row
// statistics, in the caller's CSR order whatever schedule the gather pass used: one thread per
// (edge, head), so both arrays are written as one sequential stream.  The row of an edge is found
// by bisection of row_ptr, first for the wave's first and last edge (wave-uniform), then per lane
// inside that usually one- or two-row window.
__device__ __forceinline__ int gat_row_of(const int *__restrict__ ptr, int lo, int hi, int q)
{
    while (lo < hi) {                       // largest r in [lo, hi] with ptr[r] <= q
        int mid = (lo + hi + 1) >> 1;
        if (ptr[mid] <= q) lo = mid; else hi = mid - 1;
    }
    return lo;
}
#define GAT_STASH_CHUNKS 32     // 64-element chunks per wave: the two wave-wide bisections are paid once per 2048 elements
#define GAT_STASH_UJ 4          // chunks in flight; divides GAT_STASH_CHUNKS
__global__ __launch_bounds__(FGNN_TPB) void gat_edge_stash_kernel(int N, int64_t E, int H, const int *__restrict__ ptr,
                                                                  const int *__restrict__ idx, const float *__restrict__ ar,
                                                                  const float *__restrict__ ac, const float *__restrict__ emax,
                                                                  const float *__restrict__ esum, float slope,
                                                                  float *__restrict__ e_lrelu, float *__restrict__ e_softmax)
{
    const int64_t total = E * H;
    const int64_t k0 = ((int64_t)blockIdx.x * FGNN_WPB + fg_wave()) * (64 * GAT_STASH_CHUNKS);
    if (k0 >= total) return;
    const int64_t k1 = min(k0 + 64 * GAT_STASH_CHUNKS, total);
    const int lane = fg_lane();
    const unsigned uh = (unsigned)H;
    const unsigned inv_h = (65536u + uh - 1u) / uh;          // ceil(2^16 / H)
    int qbase = fg_uni((int)(k0 / H));                       // edge of the chunk's first element
    unsigned rem = (unsigned)fg_uni((int)(k0 - (int64_t)qbase * H));
    const int qlast = fg_uni((int)((k1 - 1) / H));
    int rlo = gat_row_of(ptr, 0, N - 1, qbase);
    const int rhi = gat_row_of(ptr, rlo, N - 1, qlast);
    // GAT_STASH_UJ chunks per trip, their bisections and loads side by side: one chunk is a chain of
    // dependent loads (row bounds, source id, attn_col of the source), several in flight hide it
    constexpr int UJ = GAT_STASH_UJ;
    for (int64_t kk = k0; kk < k1; kk += 64 * UJ) {
        int q[UJ], h[UJ], lo[UJ], hi[UJ];
#pragma unroll
        for (int j = 0; j < UJ; ++j) {
            const unsigned x = rem + (unsigned)(64 * j + lane);           // < H + 64 * UJ <= 320
            const unsigned dq = (x * inv_h) >> 16;                          // = x / H for x < 1024 (H <= 64)
            h[j] = (int)(x - dq * uh);
            q[j] = min(qbase + (int)dq, qlast);
            lo[j] = rlo; hi[j] = rhi;
        }
        for (int w = rhi - rlo; w > 0; w >>= 1) {           // wave-uniform trip count: ceil(log2(window))
#pragma unroll
            for (int j = 0; j < UJ; ++j) {
                const int mid = (lo[j] + hi[j] + 1) >> 1;   // lo == hi: mid == lo, nothing changes
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
                const size_t rh = (size_t)lo[j] * H + h[j];
                const float ev = fg_lrelu(ar[rh] + ac[(size_t)src[j] * H + h[j]], slope);
                if (e_lrelu) __builtin_nontemporal_store(ev, e_lrelu + k);
                __builtin_nontemporal_store(__builtin_amdgcn_exp2f((ev - emax[rh]) * FGNN_LOG2E) * __builtin_amdgcn_rcpf(esum[rh]), e_softmax + k);
            }
        }
        rem += 64u * UJ;
        const unsigned adv = rem / uh;
        qbase += (int)adv;
        rem -= adv * uh;
        rlo = __builtin_amdgcn_readlane(lo[UJ - 1], 63);    // rows only grow along the chunks
    }
}

// The stashed attention in the ORDER OF THE BACKWARD PASS: esm[q,h] = alpha of entry q of the (col_ptr, row_ind)
// walk under the given schedule (its bucket-ordered entry order when it is XCD-aware), so that the column pass
// streams the stash instead of gathering 32 bytes per edge through `permute`.  The value stored is alpha with the sign
// bit set when the pre-activation is not positive, so the column pass needs nothing else per (destination, head) than
// delta: no 16-byte record, a quarter of the gathered bytes next to the feature rows.  Same traversal as that pass (work
// items, one wave each), pair layout: lane (u << hp_shift) | h owns (entry u of a batch, head h), gathers the three
// row statistics of (destination, h) and writes one float; a batch writes 64 consecutive floats.
__global__ __launch_bounds__(FGNN_TPB) void gat_stash_own_order_kernel(const fgnn_item *items, int n_items, const int *__restrict__ ptr,
                                                                       const int *__restrict__ idx, int H, int hp_shift,
                                                                       const float *__restrict__ ar, const float *__restrict__ ac,
                                                                       const float *__restrict__ emax, const float *__restrict__ esum,
                                                                       float slope, float *__restrict__ esm)
{
    int col, b, e, slot;
    if (!fg_get_item(items, n_items, ptr, col, b, e, slot)) return;
    const int lane = fg_lane();
    const int u = lane >> hp_shift, h = lane & ((1 << hp_shift) - 1);
    const int U = 64 >> hp_shift;                         // entries per batch
    const bool okh = h < H;
    const float ach = okh ? ac[(size_t)col * H + h] : 0.f;
    for (int c = b; c < e; c += 64) {
        const int q = c + lane;
        const int cnt = min(64, e - c);
        const int idv = idx[q < e ? q : c];
        for (int t = 0; t < cnt; t += U) {
            const int i = __builtin_amdgcn_ds_bpermute(((t + u) & 63) << 2, idv);
            if (okh && t + u < cnt) {
                const size_t rh = (size_t)(unsigned)i * H + h;
                const float ev = fg_lrelu(ar[rh] + ach, slope);
                const float al = __builtin_amdgcn_exp2f((ev - emax[rh]) * FGNN_LOG2E) * __builtin_amdgcn_rcpf(esum[rh]);
                // alpha >= 0: its sign bit carries "pre-activation positive" (clear) / "not positive" (set, -0.0 included)
                __builtin_nontemporal_store(ev > 0.f ? al : -al, esm + (size_t)(c + t + u) * H + h);
            }
        }
    }
}

// ------------------------------------------------------------------------------- backward
struct GatBwdP {
    const fgnn_item *items; int n_items;
    const int *ptr; const int *idx; const int *pos; const int *permute;
    const float4 *rec;
    const float *delta;     // own-order stash only: <g[i,h,:], out[i,h,:]> per (node, head), in place of rec
    const float *ac; const float *x; const float *g;
    const float *esm;
    float *gfeat; float *gac; float *part;
    int N, H, F, HF; float slope;
    int hp_shift;   // pair layout of the batches (gat_bwd_pair_batch): lane = (edge of the batch << hp_shift) | head
};
// Partial layout (floats): T[HF] | P[HF] | z[H]
__host__ __device__ static inline int gat_bwd_pw(int HF, int H) { return (2 * HF + H + 3) & ~3; }

// Node-wise pre-pass: delta, grad_attn_row and the packed per-(node, head) record.
template <int VEC, int R>
__global__ __launch_bounds__(FGNN_TPB) void gat_bwd_node_kernel(int N, int H, int F, int HF, const float *g, const float *out,
                                                                const float *out2, const float *cc, const float *ar,
                                                                const float *emax, const float *esum, float4 *rec, float *delta_out,
                                                                float *gar)
{
    extern __shared__ float lds[];
    int i = fg_uni((int)blockIdx.x * FGNN_WPB + fg_wave());
    if (i >= N) return;
    const int lane = fg_lane();
    float *scr = lds + fg_wave() * (64 * R);
    fg_lanemap<VEC, R> lm;
    lm.init(lane, HF, F);
    float d1[R], d2[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        d1[r] = 0.f; d2[r] = 0.f;
        if (lm.ok[r]) {
            size_t o = (size_t)i * HF + lm.eoff[r];
            fg_vec<VEC> gv, a, c;
            gv.load(g + o); a.load(out + o); c.load(out2 + o);
            d1[r] = gv.dot(a); d2[r] = gv.dot(c);
        }
    }
    float delta = fg_head_reduce<VEC, R>(scr, d1, lm, lane, H, F);
    float dd2 = fg_head_reduce<VEC, R>(scr, d2, lm, lane, H, F);
    if (lane < H) {
        size_t q = (size_t)i * H + lane;
        float s = esum[q];
        // attn_row and the maximum are stored in log2 units for the column pass; with a signed own-order stash that
        // pass only needs delta
        if (delta_out) delta_out[q] = delta;
        else rec[q] = make_float4(ar[q] * FGNN_LOG2E, emax[q] * FGNN_LOG2E, s > 0.f ? 1.f / s : 0.f, delta);
        gar[q] = dd2 - delta * cc[q];
    }
}

// The same pre-pass for rows narrower than a wave (H*F <= 128 floats in the 128-bit layout): a node takes LPN lanes (the
// power of two >= H*F/4), 64 / LPN nodes share a wave.  With one wave per node an output layer of 48 floats keeps 12 lanes
// busy and moves 576 bytes per wave (0.9 ms for 2.4 M nodes; the rows are 1.4 GB).
template <int LPN>
__global__ __launch_bounds__(FGNN_TPB) void gat_bwd_node_packed_kernel(int N, int H, int F, int HF, const float *g, const float *out,
                                                                       const float *out2, const float *cc, const float *ar,
                                                                       const float *emax, const float *esum, float4 *rec, float *delta_out,
                                                                       float *gar)
{
    constexpr int NPW = 64 / LPN;
    const int lane = fg_lane(), sub = lane % LPN;
    const int64_t node = ((int64_t)blockIdx.x * FGNN_WPB + fg_wave()) * NPW + lane / LPN;
    const bool ok = node < N && sub * 4 < HF;
    float d1 = 0.f, d2 = 0.f;
    if (ok) {
        const size_t o = (size_t)node * HF + sub * 4;
        fg_vec<4> gv, a, c;
        gv.load(g + o); a.load(out + o); c.load(out2 + o);
        d1 = gv.dot(a); d2 = gv.dot(c);
    }
    const int lph = F / 4;                                  // lanes per head
    int head = -1;                                          // the head this lane writes the results of
    if ((lph & (lph - 1)) == 0) {                           // heads are aligned groups of a power of two lanes
        for (int d = 1; d < lph; d <<= 1) { d1 += __shfl_xor(d1, d); d2 += __shfl_xor(d2, d); }
        if (ok && sub % lph == 0) head = sub / lph;
    } else {                                                // any width: one masked sum over the node's lanes per head
        const int mine = ok ? (sub * 4) / F : -1;
        float r1 = 0.f, r2 = 0.f;
        for (int h = 0; h < H; ++h) {
            float s1 = mine == h ? d1 : 0.f, s2 = mine == h ? d2 : 0.f;
#pragma unroll
            for (int d = 1; d < LPN; d <<= 1) { s1 += __shfl_xor(s1, d); s2 += __shfl_xor(s2, d); }
            if (sub == h) { r1 = s1; r2 = s2; }
        }
        d1 = r1; d2 = r2;
        if (node < N && sub < H) head = sub;                // H <= H*F/4 <= LPN
    }
    if (head >= 0) {
        const size_t q = (size_t)node * H + head;
        const float s = esum[q];
        if (delta_out) delta_out[q] = d1;
        else rec[q] = make_float4(ar[q] * FGNN_LOG2E, emax[q] * FGNN_LOG2E, s > 0.f ? 1.f / s : 0.f, d1);
        gar[q] = d2 - d1 * cc[q];
    }
}

// Writes grad_feat[col] = T and grad_attn_col[col,h] = <x[col,h,:], slope*T + (1-slope)*P> - z[h].
// z[r] is held by every lane of head hd[r]; scr is wave-private LDS of 64*R + 64 floats.
template <int VEC, int R>
__device__ __forceinline__ void gat_bwd_finish(const GatBwdP &p, int col, int lane, float *scr, const fg_lanemap<VEC, R> &lm,
                                               fg_vec<VEC> (&T)[R], fg_vec<VEC> (&P)[R], const float (&z)[R])
{
    float d[R];
    float *zs = scr + 64 * R;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        d[r] = 0.f;
        if (lm.ok[r]) {
            size_t o = (size_t)col * p.HF + lm.eoff[r];
            T[r].store_nt(p.gfeat + o);
            fg_vec<VEC> g2 = T[r].lin(p.slope, 1.f - p.slope, P[r]);
            fg_vec<VEC> xv; xv.load(p.x + o);
            d[r] = xv.dot(g2);
            if (lm.eoff[r] % p.F == 0) zs[lm.hd[r]] = z[r];
        }
    }
    float dot = fg_head_reduce<VEC, R>(scr, d, lm, lane, p.H, p.F);
    if (lane < p.H) p.gac[(size_t)col * p.H + lane] = dot - zs[lane];
}

// One batch of UB edges of the backward column pass.  Every lane reads the 16-byte record
// (attn_row, max, 1/sum, delta) of the head its features belong to (the first two in log2 units)
// and recomputes alpha itself.
// STASH: 0 = alpha recomputed from the record; 1 = alpha read from a stash in the caller's order (through permute), the
// sign of the pre-activation from attn_row + attn_col; 2 = signed alpha read from a stash in this pass's own order.
template <int VEC, int R, int STASH, bool FULL, int UB, bool TAIL, bool SLE1>
__device__ __forceinline__ void gat_bwd_batch(const GatBwdP &p, const fg_lanemap<VEC, R> &lm, const uint32_t (&boff)[R],
                                              const uint32_t (&roff)[R], const uint32_t (&hoff)[R], int idv, int posv, int t, int cnt,
                                              const float (&ach)[R], float (&z)[R], fg_vec<VEC> (&T)[R], fg_vec<VEC> (&P)[R])
{
    fg_vec<VEC> ld[UB][R];
    float4 rc[UB][R];
    const size_t row_bytes = (size_t)p.HF * sizeof(float), rec_bytes = (size_t)p.H * sizeof(float4), sc_bytes = (size_t)p.H * sizeof(float);
#pragma unroll
    for (int u = 0; u < UB; ++u) {
        size_t i = (size_t)(unsigned)__builtin_amdgcn_readlane(idv, t + u);
        const char *base = (const char *)p.g + i * row_bytes;
        const char *rb = (const char *)p.rec + i * rec_bytes;
        const char *db = (const char *)p.delta + i * sc_bytes;
        size_t pos = STASH ? (size_t)(unsigned)__builtin_amdgcn_readlane(posv, t + u) * sc_bytes : 0;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (FULL || lm.ok[r]) {
                ld[u][r].load_off(base, boff[r]);
                if (STASH == 2) rc[u][r] = make_float4(0.f, *(const float *)((const char *)p.esm + pos + hoff[r]), 0.f, *(const float *)(db + hoff[r]));
                else rc[u][r] = *(const float4 *)(rb + roff[r]);
                if (STASH == 1) rc[u][r].y = *(const float *)((const char *)p.esm + pos + hoff[r]);
            } else {
                ld[u][r].zero();
                rc[u][r] = make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
    }
#pragma unroll
    for (int u = 0; u < UB; ++u) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float ev, al;
            // stash variants: alpha comes from the stash; only the sign of the pre-activation is still
            // needed, and that is the sign of attn_row + attn_col (no second per-edge gather)
            if (STASH == 2) { ev = __float_as_int(rc[u][r].y) >= 0 ? 1.f : -1.f; al = fabsf(rc[u][r].y); }
            else if (STASH == 1) { ev = fmaf(ach[r], FGNN_LOG2E, rc[u][r].x); al = rc[u][r].y; }
            else { ev = fg_lrelu_t<SLE1>(fmaf(ach[r], FGNN_LOG2E, rc[u][r].x), p.slope); al = __builtin_amdgcn_exp2f(ev - rc[u][r].y) * rc[u][r].z; }
            if (TAIL) al = ((t + u) < cnt) ? al : 0.f;
            const bool pos_e = ev > 0.f;
            T[r].fma(al, ld[u][r]);
            P[r].fma(pos_e ? al : 0.f, ld[u][r]);
            z[r] = fmaf(pos_e ? al : al * p.slope, rc[u][r].w, z[r]);
        }
    }
}

// The same batch with the attention weights formed in a PAIR layout: lane (u << hp_shift) | h owns
// (edge u of the batch, head h), reads that one 16-byte record and computes alpha once; the feature
// lanes then fetch alpha of (their edge, their head) with ds_bpermute.  Against gat_bwd_batch, where
// every lane reads a record per edge, this takes the record reads from one L1 pass per edge (as costly
// as the feature row itself) to one per batch, and the exp / LeakyReLU arithmetic likewise.
// pr: per-lane state of the pair layout (u, h, whether the lane owns a pair, attn_col of (col, h), z).
struct GatPair { int u, h; bool ok; float ach, z; };
struct GatPairRec { float4 rc; float esm; };
// The record (and stashed alpha) of the lane's pair in the batch that starts at entry t of the chunk.
// Issued one batch ahead of its use, so that the feature-row loads of a batch never wait behind it.
template <int STASH>
__device__ __forceinline__ GatPairRec gat_bwd_pair_fetch(const GatBwdP &p, const GatPair &pr, int idv, int posv, int t, int cnt)
{
    const int eu = (t + pr.u) & 63;
    const bool live = pr.ok && t + pr.u < cnt;
    // (lane exchanges stay outside divergent code: a lane that is switched off cannot be read)
    const int ip = __builtin_amdgcn_ds_bpermute(eu << 2, idv);
    const int pp = STASH ? __builtin_amdgcn_ds_bpermute(eu << 2, posv) : 0;
    GatPairRec f;
    f.rc = make_float4(0.f, 0.f, 0.f, 0.f);
    f.esm = 0.f;
    if (live) {
        if (STASH == 2) f.rc.w = p.delta[(size_t)(unsigned)ip * p.H + pr.h];
        else f.rc = p.rec[(size_t)(unsigned)ip * p.H + pr.h];
        if (STASH) f.esm = __builtin_nontemporal_load(p.esm + (size_t)(unsigned)pp * p.H + pr.h);     // read once
    }
    return f;
}
template <int VEC, int R, int STASH, bool FULL, int UB, bool SLE1>
__device__ __forceinline__ void gat_bwd_pair_batch(const GatBwdP &p, const fg_lanemap<VEC, R> &lm, const uint32_t (&boff)[R],
                                                   int idv, int posv, int t, int cnt, GatPair &pr, GatPairRec &cur,
                                                   fg_vec<VEC> (&T)[R], fg_vec<VEC> (&P)[R])
{
    GatPairRec nxt;
    nxt.rc = make_float4(0.f, 0.f, 0.f, 0.f); nxt.esm = 0.f;
    if (t + UB < cnt) nxt = gat_bwd_pair_fetch<STASH>(p, pr, idv, posv, t + UB, cnt);      // wave-uniform
    fg_vec<VEC> ld[UB][R];
    const uint32_t row_bytes = (uint32_t)p.HF * 4u;
    uint32_t bo[R];
#pragma unroll
    for (int r = 0; r < R; ++r) bo[r] = fg_pin(boff[r]);
#pragma unroll
    for (int u = 0; u < UB; ++u) {
        uint64_t i = (uint64_t)(uint32_t)__builtin_amdgcn_readlane(idv, (t + u) & 63);      // past the chunk: any valid row, weight 0
        fg_gptr base = fg_uniform_ptr((const char *)p.g + i * row_bytes);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (FULL || lm.ok[r]) ld[u][r].load_off(base, bo[r]); else ld[u][r].zero();
        }
    }
    const float4 rc = cur.rc;
    float ev, al;
    if (STASH == 2) { ev = __float_as_int(cur.esm) >= 0 ? 1.f : -1.f; al = fabsf(cur.esm); }
    else if (STASH == 1) { ev = fmaf(pr.ach, FGNN_LOG2E, rc.x); al = cur.esm; }
    else { ev = fg_lrelu_t<SLE1>(fmaf(pr.ach, FGNN_LOG2E, rc.x), p.slope); al = __builtin_amdgcn_exp2f(ev - rc.y) * rc.z; }
    al = (pr.ok && t + pr.u < cnt) ? al : 0.f;
    pr.z = fmaf(ev > 0.f ? al : al * p.slope, rc.w, pr.z);
    // alpha >= 0, so one exchange carries both weights: the sign says whether the pre-activation was positive
    const float als = ev > 0.f ? al : -al;
#pragma unroll
    for (int u = 0; u < UB; ++u) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int src = ((u << p.hp_shift) + lm.hd[r]) << 2;
            const float a = __int_as_float(__builtin_amdgcn_ds_bpermute(src, __float_as_int(als)));
            T[r].fma(fabsf(a), ld[u][r]);
            P[r].fma(fg_relu_bits(a), ld[u][r]);
        }
    }
    cur = nxt;
}

template <int VEC, int R, int STASH, bool FULL, bool SLE1, bool PAIR>
__global__ __launch_bounds__(FGNN_TPB) void gat_bwd_kernel(GatBwdP p)
{
    extern __shared__ float lds[];
    int col, b, e, slot;
    if (!fg_get_item(p.items, p.n_items, p.ptr, col, b, e, slot)) return;
    const int lane = fg_lane();
    const int H = p.H;
    float *scr = lds + fg_wave() * (64 * R + 64);
    fg_lanemap<VEC, R> lm;
    lm.init(lane, p.HF, p.F);

    fg_vec<VEC> T[R], P[R];
    float ach[R], z[R];
    uint32_t boff[R], roff[R], hoff[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        T[r].zero(); P[r].zero(); z[r] = 0.f;
        ach[r] = p.ac[(size_t)col * H + lm.hd[r]];
        boff[r] = (uint32_t)lm.eoff[r] * 4u;
        roff[r] = (uint32_t)lm.hd[r] * 16u;
        hoff[r] = (uint32_t)lm.hd[r] * 4u;
    }

    constexpr int U = (R >= 8) ? 1 : (PAIR || R > 2 ? 8 : 4) / R;      // as in gat_fwd_kernel
    GatPair pr;
    pr.u = lane >> p.hp_shift; pr.h = lane & ((1 << p.hp_shift) - 1);
    pr.ok = PAIR && pr.h < H && pr.u < U;
    pr.ach = pr.ok ? p.ac[(size_t)col * H + pr.h] : 0.f;
    pr.z = 0.f;
    for (int c = b; c < e; c += 64) {
        int q = c + lane;
        int cnt = min(64, e - c);
        int qq = q < e ? q : c;
        int idv = p.idx[qq];
        int posv = STASH ? (p.permute ? p.permute[p.pos ? p.pos[qq] : qq] : qq) : 0;      // no permute: the stash is in this pass's own entry order
        int t = 0;
        if constexpr (PAIR) {
            GatPairRec cur = gat_bwd_pair_fetch<STASH>(p, pr, idv, posv, 0, cnt);
            for (; t + U <= cnt; t += U) gat_bwd_pair_batch<VEC, R, STASH, FULL, U, SLE1>(p, lm, boff, idv, posv, t, cnt, pr, cur, T, P);
            if constexpr (U >= 4) {
                if (cnt - t > U / 2) gat_bwd_pair_batch<VEC, R, STASH, FULL, U, SLE1>(p, lm, boff, idv, posv, t, cnt, pr, cur, T, P);
                else if (cnt - t > 0) gat_bwd_pair_batch<VEC, R, STASH, FULL, U / 2, SLE1>(p, lm, boff, idv, posv, t, cnt, pr, cur, T, P);
            } else {
                if (cnt - t > 0) gat_bwd_pair_batch<VEC, R, STASH, FULL, U, SLE1>(p, lm, boff, idv, posv, t, cnt, pr, cur, T, P);
            }
        } else {
            for (; t + U <= cnt; t += U) gat_bwd_batch<VEC, R, STASH, FULL, U, false, SLE1>(p, lm, boff, roff, hoff, idv, posv, t, cnt, ach, z, T, P);
            if constexpr (U >= 4) {
                if (cnt - t > U / 2) gat_bwd_batch<VEC, R, STASH, FULL, U, true, SLE1>(p, lm, boff, roff, hoff, idv, posv, t, cnt, ach, z, T, P);
                else if (cnt - t > 0) gat_bwd_batch<VEC, R, STASH, FULL, U / 2, true, SLE1>(p, lm, boff, roff, hoff, idv, posv, t, cnt, ach, z, T, P);
            } else {
                if (cnt - t > 0) gat_bwd_batch<VEC, R, STASH, FULL, U, true, SLE1>(p, lm, boff, roff, hoff, idv, posv, t, cnt, ach, z, T, P);
            }
        }
    }
    if constexpr (PAIR) {
        // z of head h: the sum over the edge slots of the pair layout, handed to the lanes of that head
        float zt = pr.z;
        for (int sft = 1 << p.hp_shift; sft < 64; sft <<= 1) zt += fg_bperm(zt, lane ^ sft);
#pragma unroll
        for (int r = 0; r < R; ++r) z[r] = fg_bperm(zt, lm.hd[r]);
    }

    if (slot < 0) {
        gat_bwd_finish<VEC, R>(p, col, lane, scr, lm, T, P, z);
    } else {
        float *pp = p.part + (size_t)slot * gat_bwd_pw(p.HF, H);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (!(FULL || lm.ok[r])) continue;
            T[r].store_nt(pp + lm.eoff[r]);
            P[r].store_nt(pp + p.HF + lm.eoff[r]);
            if (lm.eoff[r] % p.F == 0) pp[2 * p.HF + lm.hd[r]] = z[r];
        }
    }
}

// The column pass for rows narrower than a wave: G entries of the column per load instruction
// (see gat_fwd_packed_kernel); T, P and z are plain sums, so the groups are added by a butterfly.
template <int G, int STASH, bool SLE1, bool PAIR, int U = 8>
__device__ __forceinline__ void gat_bwd_packed_item(const GatBwdP &p, int n_head, float *lds)
{
    int col, b, e, slot;
    if (!fg_get_item(p.items, n_head, p.ptr, col, b, e, slot)) return;
    const int lane = fg_lane();
    const int H = p.H;
    float *scr = lds + fg_wave() * (64 + 64);
    fg_packmap<G> pm;
    pm.init(lane, p.HF, p.F);
    fg_vec<4> T, P;
    T.zero(); P.zero();
    float z = 0.f;
    const float ach = p.ac[(size_t)col * H + pm.hd];
    // U: load instructions in flight
    // PAIR: the attention weights are formed in the pair layout of gat_bwd_pair_batch, one lane per
    // (entry of the batch of 8*G, head)
    GatPair pr;
    pr.u = lane >> p.hp_shift; pr.h = lane & ((1 << p.hp_shift) - 1);
    pr.ok = PAIR && pr.h < H && pr.u < U * G;
    pr.ach = pr.ok ? p.ac[(size_t)col * H + pr.h] : 0.f;
    pr.z = 0.f;
    for (int c = b; c < e; c += 64) {
        int q = c + lane;
        int cnt = min(64, e - c);
        int qq = q < e ? q : c;
        int idv = p.idx[qq];
        int posv = STASH ? (p.permute ? p.permute[p.pos ? p.pos[qq] : qq] : qq) : 0;
        GatPairRec cur;
        cur.rc = make_float4(0.f, 0.f, 0.f, 0.f); cur.esm = 0.f;
        if constexpr (PAIR) cur = gat_bwd_pair_fetch<STASH>(p, pr, idv, posv, 0, cnt);
        for (int t = 0; t < cnt; t += U * G) {
            fg_vec<4> ld[U];
            if constexpr (PAIR) {
                GatPairRec nxt;
                nxt.rc = make_float4(0.f, 0.f, 0.f, 0.f); nxt.esm = 0.f;
                if (t + U * G < cnt) nxt = gat_bwd_pair_fetch<STASH>(p, pr, idv, posv, t + U * G, cnt);     // wave-uniform
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int ei = t + u * G + pm.grp;
                    const size_t i = (size_t)(unsigned)__builtin_amdgcn_ds_bpermute((ei & 63) << 2, idv);
                    if (ei < cnt && pm.ok) ld[u].load(p.g + i * p.HF + pm.eoff); else ld[u].zero();
                }
                const float4 rc = cur.rc;
                float ev, al;
                if (STASH == 2) { ev = __float_as_int(cur.esm) >= 0 ? 1.f : -1.f; al = fabsf(cur.esm); }
                else if (STASH == 1) { ev = fmaf(pr.ach, FGNN_LOG2E, rc.x); al = cur.esm; }
                else { ev = fg_lrelu_t<SLE1>(fmaf(pr.ach, FGNN_LOG2E, rc.x), p.slope); al = __builtin_amdgcn_exp2f(ev - rc.y) * rc.z; }
                al = (pr.ok && t + pr.u < cnt) ? al : 0.f;
                pr.z = fmaf(ev > 0.f ? al : al * p.slope, rc.w, pr.z);
                const float als = ev > 0.f ? al : -al;      // the sign carries "pre-activation positive"
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int src = (((u * G + pm.grp) << p.hp_shift) + pm.hd) << 2;
                    const float a = __int_as_float(__builtin_amdgcn_ds_bpermute(src, __float_as_int(als)));
                    T.fma(fabsf(a), ld[u]);
                    P.fma(fg_relu_bits(a), ld[u]);
                }
                cur = nxt;
                continue;
            }
            float4 rc[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ei = t + u * G + pm.grp;
                const size_t i = (size_t)(unsigned)__builtin_amdgcn_ds_bpermute((ei & 63) << 2, idv);
                const size_t pos = STASH ? (size_t)(unsigned)__builtin_amdgcn_ds_bpermute((ei & 63) << 2, posv) : 0;
                if (ei < cnt && pm.ok) {
                    ld[u].load(p.g + i * p.HF + pm.eoff);
                    if (STASH == 2) rc[u] = make_float4(0.f, p.esm[pos * H + pm.hd], 0.f, p.delta[i * H + pm.hd]);
                    else rc[u] = p.rec[i * H + pm.hd];
                    if (STASH == 1) rc[u].y = p.esm[pos * H + pm.hd];
                } else {
                    ld[u].zero();
                    rc[u] = make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float ev, al;
                if (STASH == 2) { ev = __float_as_int(rc[u].y) >= 0 ? 1.f : -1.f; al = fabsf(rc[u].y); }
                else if (STASH == 1) { ev = fmaf(ach, FGNN_LOG2E, rc[u].x); al = rc[u].y; }
                else { ev = fg_lrelu_t<SLE1>(fmaf(ach, FGNN_LOG2E, rc[u].x), p.slope); al = __builtin_amdgcn_exp2f(ev - rc[u].y) * rc[u].z; }
                al = ((t + u * G + pm.grp) < cnt && pm.ok) ? al : 0.f;
                const bool pos_e = ev > 0.f;
                T.fma(al, ld[u]);
                P.fma(pos_e ? al : 0.f, ld[u]);
                z = fmaf(pos_e ? al : al * p.slope, rc[u].w, z);
            }
        }
    }
    fg_pack_reduce<G>(T, lane);
    fg_pack_reduce<G>(P, lane);
    if constexpr (PAIR) {
        float zt = pr.z;
        for (int sft = 1 << p.hp_shift; sft < 64; sft <<= 1) zt += fg_bperm(zt, lane ^ sft);
        z = fg_bperm(zt, pm.hd);
    } else {
#pragma unroll
        for (int step = 64 / G; step < 64; step <<= 1) z += fg_bperm(z, lane ^ step);
    }
    fg_lanemap<4, 1> lm;
    lm.eoff[0] = pm.eoff; lm.hd[0] = pm.hd; lm.ok[0] = pm.ok && pm.grp == 0;
    if (slot < 0) {
        fg_vec<4> Ts[1] = {T}, Ps[1] = {P};
        const float zs[1] = {z};
        gat_bwd_finish<4, 1>(p, col, lane, scr, lm, Ts, Ps, zs);
    } else if (lm.ok[0]) {
        float *pp = p.part + (size_t)slot * gat_bwd_pw(p.HF, H);
        T.store_nt(pp + pm.eoff);
        P.store_nt(pp + p.HF + pm.eoff);
        if (pm.eoff % p.F == 0) pp[2 * p.HF + pm.hd] = z;
    }
}

// The column pass with the lane groups on different items (see gat_fwd_rowpack_items).  T, P and z of an item stay inside
// its group; the per-head dot product of the epilogue is reduced inside the group as well (no LDS).
template <int G, int STASH, bool SLE1>
__device__ __forceinline__ void gat_bwd_rowpack_items(const GatBwdP &p, int bucketed, int first, int w)
{
    constexpr int LPR = 64 / G, U = 4;
    const int lane = fg_lane();
    const int H = p.H;
    fg_packmap<G> pm;
    pm.init(lane, p.HF, p.F);
    const int sl = lane & (LPR - 1), gbase = lane - sl;
    const int it = fg_group_slot(G, pm.grp, bucketed, first, w);
    int col = -1, b = 0, e = 0, slot = -1;
    if (it < p.n_items) {
        if (p.items) { const fgnn_item q = p.items[it]; col = q.row; b = q.begin; e = q.end; slot = q.slot; }
        else { col = it; b = p.ptr[it]; e = p.ptr[it + 1]; }
    }
    if (col < 0) { b = 0; e = 0; }
    if (__builtin_amdgcn_ballot_w64(col >= 0) == 0ull) return;
    fg_vec<4> T, P;
    T.zero(); P.zero();
    float z = 0.f;
    const float ach = col >= 0 ? p.ac[(size_t)col * H + pm.hd] : 0.f;
    for (int c = b; __builtin_amdgcn_ballot_w64(c < e) != 0ull; c += LPR) {
        const int cnt = min(LPR, e - c);                              // <= 0: this group is done
        int idv = 0, posv = 0;
        if (c < e) {
            const int qq = c + sl < e ? c + sl : c;                   // idle lanes repeat a valid entry
            idv = p.idx[qq];
            if (STASH) posv = p.permute ? p.permute[p.pos ? p.pos[qq] : qq] : qq;
        }
        for (int t = 0; __builtin_amdgcn_ballot_w64(t < cnt) != 0ull; t += U) {
            fg_vec<4> ld[U];
            float4 rc[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ei = t + u, src = (gbase + (ei & (LPR - 1))) << 2;
                const size_t i = (size_t)(unsigned)__builtin_amdgcn_ds_bpermute(src, idv);
                const size_t pos = STASH ? (size_t)(unsigned)__builtin_amdgcn_ds_bpermute(src, posv) : 0;
                if (ei < cnt && pm.ok) {
                    ld[u].load(p.g + i * p.HF + pm.eoff);
                    if (STASH == 2) rc[u] = make_float4(0.f, p.esm[pos * H + pm.hd], 0.f, p.delta[i * H + pm.hd]);
                    else rc[u] = p.rec[i * H + pm.hd];
                    if (STASH == 1) rc[u].y = p.esm[pos * H + pm.hd];
                } else {
                    ld[u].zero();
                    rc[u] = make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float ev, al;
                if (STASH == 2) { ev = __float_as_int(rc[u].y) >= 0 ? 1.f : -1.f; al = fabsf(rc[u].y); }
                else if (STASH == 1) { ev = fmaf(ach, FGNN_LOG2E, rc[u].x); al = rc[u].y; }
                else { ev = fg_lrelu_t<SLE1>(fmaf(ach, FGNN_LOG2E, rc[u].x), p.slope); al = __builtin_amdgcn_exp2f(ev - rc[u].y) * rc[u].z; }
                al = (t + u < cnt && pm.ok) ? al : 0.f;
                const bool pos_e = ev > 0.f;
                T.fma(al, ld[u]);
                P.fma(pos_e ? al : 0.f, ld[u]);
                z = fmaf(pos_e ? al : al * p.slope, rc[u].w, z);
            }
        }
    }
    // epilogue of gat_bwd_finish, inside the group: every lane of a head holds that head's z
    const bool whole = col >= 0 && slot < 0;
    float d = 0.f;
    if (whole && pm.ok) {
        const size_t o = (size_t)col * p.HF + pm.eoff;
        T.store_nt(p.gfeat + o);
        fg_vec<4> g2 = T.lin(p.slope, 1.f - p.slope, P);
        fg_vec<4> xv; xv.load(p.x + o);
        d = xv.dot(g2);
    }
    const int lph = p.F / 4;                                          // lanes per head
    if ((lph & (lph - 1)) == 0) {                                     // heads are aligned runs of a power of two lanes
        for (int s = 1; s < lph; s <<= 1) d += __shfl_xor(d, s);
        if (whole && pm.ok && sl % lph == 0) p.gac[(size_t)col * H + pm.hd] = d - z;
    } else {                                                          // any width: one masked sum over the group per head
        float r = 0.f;
        for (int h = 0; h < H; ++h) {
            float s1 = (pm.ok && pm.hd == h) ? d : 0.f;
#pragma unroll
            for (int s = 1; s < LPR; s <<= 1) s1 += __shfl_xor(s1, s);
            if (sl == h) r = s1;
        }
        const float zh = fg_bperm(z, gbase + min(sl, H - 1) * lph);   // z of head sl, from that head's first lane
        if (whole && sl < H) p.gac[(size_t)col * H + sl] = r - zh;
    }
    if (col >= 0 && slot >= 0 && pm.ok) {
        float *pp = p.part + (size_t)slot * gat_bwd_pw(p.HF, H);
        T.store_nt(pp + pm.eoff);
        P.store_nt(pp + p.HF + pm.eoff);
        if (pm.eoff % p.F == 0) pp[2 * p.HF + pm.hd] = z;
    }
}

template <int G, int STASH, bool SLE1, bool PAIR>
__global__ __launch_bounds__(FGNN_TPB) void gat_bwd_packed_kernel(GatBwdP p)
{
    extern __shared__ float lds[];
    gat_bwd_packed_item<G, STASH, SLE1, PAIR>(p, p.n_items, lds);
}
// Head of the list a wave per item, the rest a lane group per item, in one launch (see gat_fwd_mixed_kernel).
template <int G, int STASH, bool SLE1, bool PAIR>
__global__ __launch_bounds__(FGNN_TPB) void gat_bwd_mixed_kernel(GatBwdP p, int bucketed, int first, unsigned head_blocks)
{
    extern __shared__ float lds[];
    if (blockIdx.x < head_blocks) gat_bwd_packed_item<G, STASH, SLE1, PAIR, 4>(p, first, lds);
    else gat_bwd_rowpack_items<G, STASH, SLE1>(p, bucketed, first, (int)(blockIdx.x - head_blocks));
}

template <int VEC, int R>
__global__ __launch_bounds__(FGNN_TPB) void gat_bwd_merge_kernel(GatBwdP p, const fgnn_split *split, int n_split)
{
    extern __shared__ float lds[];
    int w = fg_uni((int)blockIdx.x * FGNN_WPB + fg_wave());
    if (w >= n_split) return;
    fgnn_split sp = split[w];
    const int col = fg_uni(sp.row), first = fg_uni(sp.first_slot), nseg = fg_uni(sp.nseg);
    const int lane = fg_lane();
    const int H = p.H, HF = p.HF;
    const int pw = gat_bwd_pw(HF, H);
    float *scr = lds + fg_wave() * (64 * R + 64);
    fg_lanemap<VEC, R> lm;
    lm.init(lane, HF, p.F);
    fg_vec<VEC> T[R], P[R];
    float z[R];
#pragma unroll
    for (int r = 0; r < R; ++r) { T[r].zero(); P[r].zero(); z[r] = 0.f; }
    const float *base = p.part + (size_t)first * pw;
    for (int g = 0; g < nseg; ++g) {
        const float *pg = base + (size_t)g * pw;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (!lm.ok[r]) continue;
            fg_vec<VEC> t, q;
            t.load(pg + lm.eoff[r]); q.load(pg + HF + lm.eoff[r]);
            T[r].add(t); P[r].add(q);
            z[r] += pg[2 * HF + lm.hd[r]];
        }
    }
    gat_bwd_finish<VEC, R>(p, col, lane, scr, lm, T, P, z);
}

// ------------------------------------------------------------------------------- host

// idx: the index array the operator was given (an XCD-aware schedule must have been built from it)
static int check_sched(const fgnn_schedule_t *s, const int32_t *ptr, const int32_t *idx, int n, int64_t E, const char *what)
{
    if (!s) return 0;
    FGNN_REQUIRE(s->ptr_dev == ptr && s->n_rows == n && s->n_edges == E, FGNN_ERR_SCHEDULE,
                 "%s: schedule was built for another pointer array (n_rows %d vs %d, edges %lld vs %lld)", what,
                 s->n_rows, n, (long long)s->n_edges, (long long)E);
    if (s->n_buckets > 0)
        FGNN_REQUIRE(s->idx_src_dev == idx, FGNN_ERR_SCHEDULE, "%s: XCD-aware schedule was built from another index array", what);
    return 0;
}

static int gat_common_checks(const char *fn, int N, int64_t E, int H, int F)
{
    FGNN_REQUIRE(N >= 0 && E >= 0 && H >= 1 && F >= 1, FGNN_ERR_SHAPE, "%s: bad sizes N=%d E=%lld H=%d F=%d", fn, N, (long long)E, H, F);
    FGNN_REQUIRE(E <= 2147483647LL, FGNN_ERR_LIMIT, "%s: E=%lld exceeds int32 positions", fn, (long long)E);
    FGNN_REQUIRE(H <= 64, FGNN_ERR_LIMIT, "%s: H=%d > 64 heads unsupported", fn, H);
    FGNN_REQUIRE(F <= 1024, FGNN_ERR_LIMIT, "%s: F=%d > 1024 floats per head unsupported", fn, F);
    return 0;
}

// Rows of more than 1024 floats (the reference launches its recompute and stash kernels for any number of heads of up to
// 1024 floats each, src/fused_gat/fused_gat_SM.cu:518-522, :843-847) are served in passes over groups of heads: scores,
// row statistics and outputs of different heads never meet, so a pass copies the slices of `hg` heads of the node-sized
// arrays into contiguous buffers of the workspace, runs the ordinary entry on them and copies its results back.
__global__ __launch_bounds__(256) void copy2d_kernel(const float *__restrict__ src, size_t src_ld, float *__restrict__ dst, size_t dst_ld,
                                                     size_t rows, int cols)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * (size_t)cols) return;
    const size_t r = i / (size_t)cols, c = i - r * (size_t)cols;
    dst[r * dst_ld + c] = src[r * src_ld + c];
}
static int copy2d(const float *src, size_t src_ld, float *dst, size_t dst_ld, size_t rows, int cols, hipStream_t st)
{
    const size_t n = rows * (size_t)cols;
    if (n == 0) return 0;
    FGNN_REQUIRE((n + 255) / 256 <= 2147483647ULL, FGNN_ERR_LIMIT, "head-group copy: too many elements");
    hipLaunchKernelGGL(copy2d_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, src, src_ld, dst, dst_ld, rows, cols);
    return fgnn_launch_status("copy2d_kernel");
}
static inline int gat_group_heads(int H, int F) { return (int64_t)H * F <= 1024 ? H : std::max(1, 1024 / F); }
static inline size_t gat_nf_bytes(int N, int hg, int F) { return fgnn_align256((size_t)N * hg * F * sizeof(float)); }
static inline size_t gat_nh_bytes(int N, int hg) { return fgnn_align256((size_t)N * hg * sizeof(float)); }

extern "C" size_t fgnn_gat_forward_workspace_bytes(const fgnn_schedule_t *sched, int H, int F)
{
    if (!sched) return 0;
    const int hg = gat_group_heads(H, F);
    size_t b = (size_t)sched->n_partials * gat_fwd_pw(hg * F, hg, true) * sizeof(float);
    if (hg < H)        // slices of in_feat, out, out2 and of attn_row, attn_col, edge_max, edge_sum, c
        b = fgnn_align256(b) + 3 * gat_nf_bytes(sched->n_rows, hg, F) + 5 * gat_nh_bytes(sched->n_rows, hg);
    return b;
}

// The stashed per-edge tensors of the stash variants in CSR order, from the row statistics (no dependence on F).
static int gat_stash_csr_order(int N, int64_t E, int H, const int32_t *row_ptr, const int32_t *col_ind, const float *attn_row,
                               const float *attn_col, const float *edge_max, const float *edge_sum, float slope, float *e_lrelu,
                               float *e_softmax, hipStream_t st)
{
    if (!e_softmax || E == 0) return 0;
    const int64_t waves = (E * H + 64 * GAT_STASH_CHUNKS - 1) / (64 * GAT_STASH_CHUNKS);
    hipLaunchKernelGGL(gat_edge_stash_kernel, dim3((unsigned)((waves + FGNN_WPB - 1) / FGNN_WPB)), dim3(FGNN_TPB), 0, st, N, E, H, row_ptr,
                       col_ind, attn_row, attn_col, edge_max, edge_sum, slope, e_lrelu, e_softmax);
    return fgnn_launch_status("gat_edge_stash_kernel");
}

// Rows narrower than a wave on graphs of short rows: the short items of the work list go G to a wave, every lane group on an
// item of its own (gat_fwd_rowpack_items); with a wave per item, an item of two dozen entries fills one batch of 8*G loads at
// best, and the wave then spends as long combining its groups as gathering.  Measured on R-MAT graphs, forward + backward of
// a layer: 1 x 48 floats 9.0 -> 7.6 ms at 2.4 M nodes x 26 entries per row, 9.9 -> 8.3 ms at 48 entries, 7.7 -> 7.3 ms at 128,
// but 4.6 -> 4.8 ms at 492 (there the gathered rows hit L2 and the pair layout's single pass over the scores wins); 1 x 16
// floats at 1 M nodes 3.2 -> 2.2 ms; 4 x 32 floats (two groups) 15.7 -> 15.1 ms at 2.4 M nodes, 1.02 -> 0.99 ms at 169 k
// nodes, 13.9 -> 14.5 ms at 128 entries per row.
static inline bool gat_rowpack_wanted(int pack, int64_t E, int N)
{
    return E < (pack >= 4 ? 256 : 64) * (int64_t)N;
}
static int gat_forward_launch(int N, int64_t E, int H, int F, const float *attn_row, const float *attn_col,
                              const int32_t *row_ptr, const int32_t *col_ind, float slope, const float *in_feat,
                              float *out, float *edge_max, float *edge_sum, float *aux_out2, float *aux_c,
                              float *e_lrelu, float *e_softmax, const fgnn_schedule_t *sched, void *workspace,
                              size_t workspace_bytes, hipStream_t st)
{
    const int HF = H * F;
    const bool aux = aux_out2 != nullptr;
    bool aligned = fgnn_aligned16(in_feat) && fgnn_aligned16(out) && (!aux || fgnn_aligned16(aux_out2)) && fgnn_aligned16(workspace);
    fgnn_rowcfg cfg;
    FGNN_REQUIRE(fgnn_pick_rowcfg(HF, F, aligned, &cfg), FGNN_ERR_LIMIT, "fgnn_gat_forward: unsupported row width %d", HF);
    GatFwdP p{};
    p.items = sched ? sched->items_dev : nullptr;
    p.n_items = sched ? sched->n_items : N;
    p.ptr = row_ptr; p.idx = fgnn_sched_idx(sched, col_ind); p.ar = attn_row; p.ac = attn_col; p.x = in_feat;
    p.out = out; p.emax = edge_max; p.esum = edge_sum; p.out2 = aux_out2; p.cc = aux_c;
    p.part = (float *)workspace; p.N = N; p.H = H; p.F = F; p.HF = HF; p.slope = slope;
    if (sched && sched->n_partials > 0) {
        size_t need = (size_t)sched->n_partials * gat_fwd_pw(HF, H, aux) * sizeof(float);
        FGNN_REQUIRE(workspace && workspace_bytes >= need, FGNN_ERR_WORKSPACE, "fgnn_gat_forward: workspace %zu < %zu bytes", workspace_bytes, need);
    }
    if (p.n_items == 0) return 0;
    const unsigned grid = (unsigned)((p.n_items + FGNN_WPB - 1) / FGNN_WPB);
    const size_t shm = 0;
    int rc = fgnn_dispatch_rowcfg(cfg, [&]<int VEC, int R, bool FULL>() -> int {
        const bool sle1 = slope >= 0.f && slope <= 1.f;
        const int pack = fgnn_pick_pack(cfg.vec, HF);
        if (pack > 1) {
            p.hp_shift = 0;
            while ((1 << p.hp_shift) < H) ++p.hp_shift;
            // the pair layout needs 8*G entry slots x heads (rounded up to a power of two) <= 64 lanes
            const bool pair = ((8 * pack) << p.hp_shift) <= 64 && E >= 64 * (int64_t)N;
            // the long items at the head of the list keep a wave each; the rest go G to a wave on graphs of short rows
            const int first = sched && gat_rowpack_wanted(pack, E, N) ? sched->n_wave_slots : p.n_items;
            const int bucketed = sched && sched->n_buckets > 0;
            const unsigned head_blocks = (unsigned)((first + FGNN_WPB - 1) / FGNN_WPB);      // first is a multiple of 64, or n_items
            const unsigned grid_mixed = head_blocks + fgnn_group_item_grid(p.n_items - first, pack, bucketed);
            auto launch = [&]<int G>() {
                auto go = [&]<bool PAIR>() {
                    if (first < p.n_items) {
                        if (aux && sle1) hipLaunchKernelGGL((gat_fwd_mixed_kernel<G, true, true, PAIR>), dim3(grid_mixed), dim3(FGNN_TPB), 0, st, p, bucketed, first, head_blocks);
                        else if (aux) hipLaunchKernelGGL((gat_fwd_mixed_kernel<G, true, false, PAIR>), dim3(grid_mixed), dim3(FGNN_TPB), 0, st, p, bucketed, first, head_blocks);
                        else if (sle1) hipLaunchKernelGGL((gat_fwd_mixed_kernel<G, false, true, PAIR>), dim3(grid_mixed), dim3(FGNN_TPB), 0, st, p, bucketed, first, head_blocks);
                        else hipLaunchKernelGGL((gat_fwd_mixed_kernel<G, false, false, PAIR>), dim3(grid_mixed), dim3(FGNN_TPB), 0, st, p, bucketed, first, head_blocks);
                        return;
                    }
                    if (aux && sle1) hipLaunchKernelGGL((gat_fwd_packed_kernel<G, true, true, PAIR>), dim3(grid), dim3(FGNN_TPB), 0, st, p);
                    else if (aux) hipLaunchKernelGGL((gat_fwd_packed_kernel<G, true, false, PAIR>), dim3(grid), dim3(FGNN_TPB), 0, st, p);
                    else if (sle1) hipLaunchKernelGGL((gat_fwd_packed_kernel<G, false, true, PAIR>), dim3(grid), dim3(FGNN_TPB), 0, st, p);
                    else hipLaunchKernelGGL((gat_fwd_packed_kernel<G, false, false, PAIR>), dim3(grid), dim3(FGNN_TPB), 0, st, p);
                };
                if (pair) go.template operator()<true>(); else go.template operator()<false>();
            };
            if (pack == 8) launch.template operator()<8>();
            else if (pack == 4) launch.template operator()<4>();
            else launch.template operator()<2>();
        }
        else {
            // pair layout of the scores: needs (edges per batch) x (heads rounded up to a power of two) <= 64 lanes.
            // It pays where the gathered rows mostly hit L2 and the L1 passes per edge are the limit (long rows:
            // 6.8 -> 6.5 ms at 115 M edges, degree 492); on short rows out of HBM its extra exchange latency
            // per batch costs a few percent, so rows averaging under 64 entries keep the per-lane form.
            constexpr int U = (R >= 8) ? 1 : 8 / R;
            p.hp_shift = 0;
            while ((1 << p.hp_shift) < H) ++p.hp_shift;
            const bool pair = (U << p.hp_shift) <= 64 && E >= 64 * (int64_t)N;
            auto launch = [&]<bool PAIR>() {
                if (aux && sle1) hipLaunchKernelGGL((gat_fwd_kernel<VEC, R, true, FULL, true, PAIR>), dim3(grid), dim3(FGNN_TPB), shm, st, p);
                else if (aux) hipLaunchKernelGGL((gat_fwd_kernel<VEC, R, true, FULL, false, PAIR>), dim3(grid), dim3(FGNN_TPB), shm, st, p);
                else if (sle1) hipLaunchKernelGGL((gat_fwd_kernel<VEC, R, false, FULL, true, PAIR>), dim3(grid), dim3(FGNN_TPB), shm, st, p);
                else hipLaunchKernelGGL((gat_fwd_kernel<VEC, R, false, FULL, false, PAIR>), dim3(grid), dim3(FGNN_TPB), shm, st, p);
            };
            if (pair) launch.template operator()<true>(); else launch.template operator()<false>();
        }
        int rc2 = fgnn_launch_status("gat_fwd_kernel");
        if (rc2) return rc2;
        if (sched && sched->n_split > 0) {
            unsigned g2 = (unsigned)((sched->n_split + FGNN_WPB - 1) / FGNN_WPB);
            if (aux) hipLaunchKernelGGL((gat_fwd_merge_kernel<VEC, R, true>), dim3(g2), dim3(FGNN_TPB), 0, st, p, sched->split_dev, sched->n_split);
            else hipLaunchKernelGGL((gat_fwd_merge_kernel<VEC, R, false>), dim3(g2), dim3(FGNN_TPB), 0, st, p, sched->split_dev, sched->n_split);
            return fgnn_launch_status("gat_fwd_merge_kernel");
        }
        return 0;
    });
    if (rc) return rc;
    return gat_stash_csr_order(N, E, H, row_ptr, col_ind, attn_row, attn_col, edge_max, edge_sum, slope, e_lrelu, e_softmax, st);
}

extern "C" int fgnn_gat_forward(int N, int64_t E, int H, int F, const float *attn_row, const float *attn_col,
                                const int32_t *row_ptr, const int32_t *col_ind, float negative_slope,
                                const float *in_feat, float *out, float *edge_max, float *edge_sum,
                                float *aux_out2, float *aux_c, float *e_lrelu, float *e_softmax,
                                const fgnn_schedule_t *sched, void *workspace, size_t workspace_bytes, void *stream)
{
    int rc = gat_common_checks("fgnn_gat_forward", N, E, H, F);
    if (rc) return rc;
    FGNN_REQUIRE(attn_row && attn_col && row_ptr && in_feat && out && edge_max && edge_sum && (col_ind || E == 0),
                 FGNN_ERR_NULL, "fgnn_gat_forward: NULL argument");
    FGNN_REQUIRE((aux_out2 == nullptr) == (aux_c == nullptr), FGNN_ERR_NULL, "fgnn_gat_forward: aux_out2 and aux_c go together");
    FGNN_REQUIRE(e_lrelu == nullptr || e_softmax != nullptr, FGNN_ERR_NULL, "fgnn_gat_forward: e_lrelu is only written together with e_softmax");
    rc = check_sched(sched, row_ptr, col_ind, N, E, "fgnn_gat_forward");
    if (rc) return rc;
    const int hmax = gat_group_heads(H, F);
    if (hmax < H) {
        FGNN_REQUIRE(sched, FGNN_ERR_SCHEDULE, "fgnn_gat_forward: rows of more than 1024 floats (H*F=%lld) need a schedule", (long long)H * F);
        const size_t need = fgnn_gat_forward_workspace_bytes(sched, H, F);
        FGNN_REQUIRE(workspace && workspace_bytes >= need, FGNN_ERR_WORKSPACE, "fgnn_gat_forward: workspace %zu < %zu bytes", workspace_bytes, need);
        FGNN_REQUIRE(fgnn_aligned16(workspace), FGNN_ERR_ALIGN, "fgnn_gat_forward: workspace not 16-byte aligned");
        hipStream_t st = (hipStream_t)stream;
        const size_t nf = gat_nf_bytes(N, hmax, F), nh = gat_nh_bytes(N, hmax), HF = (size_t)H * F;
        char *w = (char *)workspace;
        float *xg = (float *)w; w += nf;
        float *og = (float *)w; w += nf;
        float *o2g = (float *)w; w += nf;
        float *arg = (float *)w; w += nh;
        float *acg = (float *)w; w += nh;
        float *mxg = (float *)w; w += nh;
        float *smg = (float *)w; w += nh;
        float *cg = (float *)w; w += nh;
        const size_t inner = workspace_bytes - (size_t)(w - (char *)workspace);
        const bool aux = aux_out2 != nullptr;
        for (int h0 = 0; h0 < H; h0 += hmax) {
            const int hg = std::min(hmax, H - h0);
            const size_t gf = (size_t)hg * F;
            if ((rc = copy2d(attn_row + h0, H, arg, hg, N, hg, st))) return rc;
            if ((rc = copy2d(attn_col + h0, H, acg, hg, N, hg, st))) return rc;
            if ((rc = copy2d(in_feat + (size_t)h0 * F, HF, xg, gf, N, (int)gf, st))) return rc;
            rc = gat_forward_launch(N, E, hg, F, arg, acg, row_ptr, col_ind, negative_slope, xg, og, mxg, smg, aux ? o2g : nullptr,
                                    aux ? cg : nullptr, nullptr, nullptr, sched, w, inner, st);
            if (rc) return rc;
            if ((rc = copy2d(og, gf, out + (size_t)h0 * F, HF, N, (int)gf, st))) return rc;
            if ((rc = copy2d(mxg, hg, edge_max + h0, H, N, hg, st))) return rc;
            if ((rc = copy2d(smg, hg, edge_sum + h0, H, N, hg, st))) return rc;
            if (aux) {
                if ((rc = copy2d(o2g, gf, aux_out2 + (size_t)h0 * F, HF, N, (int)gf, st))) return rc;
                if ((rc = copy2d(cg, hg, aux_c + h0, H, N, hg, st))) return rc;
            }
        }
        return gat_stash_csr_order(N, E, H, row_ptr, col_ind, attn_row, attn_col, edge_max, edge_sum, negative_slope, e_lrelu, e_softmax, st);
    }
    return gat_forward_launch(N, E, H, F, attn_row, attn_col, row_ptr, col_ind, negative_slope, in_feat, out, edge_max,
                              edge_sum, aux_out2, aux_c, e_lrelu, e_softmax, sched, workspace, workspace_bytes, (hipStream_t)stream);
}

// Backward workspace: rec [N*H float4] | recompute area (out, out2 [N*HF each], c, max, sum [N*H each]) | partials

extern "C" size_t fgnn_gat_backward_workspace_bytes(int N, int H, int F, const fgnn_schedule_t *sched_csc,
                                                    const fgnn_schedule_t *sched_csr, int need_recompute)
{
    const int hg = gat_group_heads(H, F);
    if (hg < H) {      // head-group passes: the ordinary workspace of one group plus the contiguous slices
        const bool rec = (need_recompute & 1) != 0, stash = (need_recompute & 2) != 0;
        size_t b = fgnn_align256(fgnn_gat_backward_workspace_bytes(N, hg, F, sched_csc, sched_csr, need_recompute & 1));
        b += (size_t)(rec ? 3 : 5) * gat_nf_bytes(N, hg, F) + (size_t)(rec ? 6 : 7) * gat_nh_bytes(N, hg);
        if (stash && sched_csc) b += fgnn_align256((size_t)sched_csc->n_edges * hg * sizeof(float));
        return b;
    }
    need_recompute &= 1;
    size_t HF = (size_t)H * F;
    size_t b = fgnn_align256((size_t)N * H * sizeof(float4));
    if (need_recompute) {
        b += 2 * fgnn_align256((size_t)N * HF * sizeof(float)) + 3 * fgnn_align256((size_t)N * H * sizeof(float));
        b += fgnn_align256(fgnn_gat_forward_workspace_bytes(sched_csr, H, F));
    }
    if (sched_csc) b += fgnn_align256((size_t)sched_csc->n_partials * gat_bwd_pw((int)HF, H) * sizeof(float));
    return b;
}

// own_order: e_softmax is the stash of fgnn_gat_stash_own_order (entry order of this pass under sched_csc, sign bit =
// pre-activation not positive) and permute is not used; otherwise a stash is CSR-ordered and read through permute.
static int gat_backward_impl(int N, int64_t E, int H, int F, float negative_slope, const int32_t *row_ptr,
                             const int32_t *col_ind, const int32_t *col_ptr, const int32_t *row_ind,
                             const int32_t *permute, const float *e_softmax, int own_order,
                             const float *edge_max, const float *edge_sum, const float *in_feat,
                             const float *attn_row, const float *attn_col, const float *out_feat,
                             const float *aux_out2, const float *aux_c, const float *grad_out, float *grad_feat,
                             float *grad_attn_row, float *grad_attn_col, const fgnn_schedule_t *sched_csc,
                             const fgnn_schedule_t *sched_csr, void *workspace, size_t workspace_bytes, void *stream)
{
    int rc = gat_common_checks("fgnn_gat_backward", N, E, H, F);
    if (rc) return rc;
    if (own_order) permute = nullptr;
    FGNN_REQUIRE(col_ptr && (row_ind || E == 0) && edge_max && edge_sum && in_feat && attn_row && attn_col && grad_out &&
                     grad_feat && grad_attn_row && grad_attn_col,
                 FGNN_ERR_NULL, "fgnn_gat_backward: NULL argument");
    const bool stash = e_softmax != nullptr;
    FGNN_REQUIRE(!stash || own_order || permute, FGNN_ERR_NULL,
                 "fgnn_gat_backward: stashed attention needs permute (a stash in the pass's own order goes to fgnn_gat_backward_own_order)");
    FGNN_REQUIRE(!stash || own_order || fgnn_sched_has_pos(sched_csc), FGNN_ERR_SCHEDULE, "fgnn_gat_backward: stashed attention in the caller's order needs a schedule built with edge positions");
    const bool recompute = !(out_feat && aux_out2 && aux_c);
    FGNN_REQUIRE(!recompute || (row_ptr && (col_ind || E == 0)), FGNN_ERR_NULL, "fgnn_gat_backward: recomputing the forward needs row_ptr/col_ind");
    rc = check_sched(sched_csc, col_ptr, row_ind, N, E, "fgnn_gat_backward(csc)");
    if (rc) return rc;
    if (recompute) { rc = check_sched(sched_csr, row_ptr, col_ind, N, E, "fgnn_gat_backward(csr)"); if (rc) return rc; }
    const int hmax = gat_group_heads(H, F);
    FGNN_REQUIRE(hmax == H || sched_csc, FGNN_ERR_SCHEDULE, "fgnn_gat_backward: rows of more than 1024 floats (H*F=%lld) need a schedule", (long long)H * F);
    size_t need = fgnn_gat_backward_workspace_bytes(N, H, F, sched_csc, recompute ? sched_csr : nullptr, (recompute ? 1 : 0) | (stash ? 2 : 0));
    FGNN_REQUIRE(workspace && workspace_bytes >= need, FGNN_ERR_WORKSPACE, "fgnn_gat_backward: workspace %zu < %zu bytes", workspace_bytes, need);
    FGNN_REQUIRE(fgnn_aligned16(workspace), FGNN_ERR_ALIGN, "fgnn_gat_backward: workspace not 16-byte aligned");
    if (N == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    if (hmax < H) {
        // passes over groups of heads on contiguous slices (see fgnn_gat_forward_workspace_bytes)
        const size_t nf = gat_nf_bytes(N, hmax, F), nh = gat_nh_bytes(N, hmax), HFw = (size_t)H * F;
        char *w = (char *)workspace;
        auto take = [&](size_t bytes) { float *q = (float *)w; w += bytes; return q; };
        float *xg = take(nf), *gog = take(nf), *gfg = take(nf);
        float *og = recompute ? nullptr : take(nf), *o2g = recompute ? nullptr : take(nf);
        float *arg = take(nh), *acg = take(nh), *mxg = take(nh), *smg = take(nh), *garg = take(nh), *gacg = take(nh);
        float *cg = recompute ? nullptr : take(nh);
        float *esg = stash ? take(fgnn_align256((size_t)E * hmax * sizeof(float))) : nullptr;
        const size_t inner = workspace_bytes - (size_t)(w - (char *)workspace);
        for (int h0 = 0; h0 < H; h0 += hmax) {
            const int hg = std::min(hmax, H - h0);
            const size_t gf = (size_t)hg * F;
            if ((rc = copy2d(attn_row + h0, H, arg, hg, N, hg, st))) return rc;
            if ((rc = copy2d(attn_col + h0, H, acg, hg, N, hg, st))) return rc;
            if ((rc = copy2d(edge_max + h0, H, mxg, hg, N, hg, st))) return rc;
            if ((rc = copy2d(edge_sum + h0, H, smg, hg, N, hg, st))) return rc;
            if ((rc = copy2d(in_feat + (size_t)h0 * F, HFw, xg, gf, N, (int)gf, st))) return rc;
            if ((rc = copy2d(grad_out + (size_t)h0 * F, HFw, gog, gf, N, (int)gf, st))) return rc;
            if (!recompute) {
                if ((rc = copy2d(out_feat + (size_t)h0 * F, HFw, og, gf, N, (int)gf, st))) return rc;
                if ((rc = copy2d(aux_out2 + (size_t)h0 * F, HFw, o2g, gf, N, (int)gf, st))) return rc;
                if ((rc = copy2d(aux_c + h0, H, cg, hg, N, hg, st))) return rc;
            }
            if (stash && (rc = copy2d(e_softmax + h0, H, esg, hg, (size_t)E, hg, st))) return rc;
            rc = gat_backward_impl(N, E, hg, F, negative_slope, row_ptr, col_ind, col_ptr, row_ind, permute, esg, own_order, mxg, smg, xg, arg, acg,
                                   og, o2g, cg, gog, gfg, garg, gacg, sched_csc, sched_csr, w, inner, stream);
            if (rc) return rc;
            if ((rc = copy2d(gfg, gf, grad_feat + (size_t)h0 * F, HFw, N, (int)gf, st))) return rc;
            if ((rc = copy2d(garg, hg, grad_attn_row + h0, H, N, hg, st))) return rc;
            if ((rc = copy2d(gacg, hg, grad_attn_col + h0, H, N, hg, st))) return rc;
        }
        return 0;
    }
    const int HF = H * F;
    char *w = (char *)workspace;
    float4 *rec = (float4 *)w; w += fgnn_align256((size_t)N * H * sizeof(float4));
    if (recompute) {
        float *r_out = (float *)w; w += fgnn_align256((size_t)N * HF * sizeof(float));
        float *r_out2 = (float *)w; w += fgnn_align256((size_t)N * HF * sizeof(float));
        float *r_c = (float *)w; w += fgnn_align256((size_t)N * H * sizeof(float));
        float *r_max = (float *)w; w += fgnn_align256((size_t)N * H * sizeof(float));
        float *r_sum = (float *)w; w += fgnn_align256((size_t)N * H * sizeof(float));
        void *fws = w; size_t fwb = fgnn_align256(fgnn_gat_forward_workspace_bytes(sched_csr, H, F)); w += fwb;
        // the recomputation writes its own row statistics (the same values): the caller's stay read-only
        rc = gat_forward_launch(N, E, H, F, attn_row, attn_col, row_ptr, col_ind, negative_slope, in_feat, r_out,
                                r_max, r_sum, r_out2, r_c, nullptr, nullptr, sched_csr, fws, fwb, st);
        if (rc) return rc;
        out_feat = r_out; aux_out2 = r_out2; aux_c = r_c; edge_max = r_max; edge_sum = r_sum;
    }
    float *part = (float *)w;

    bool aligned = fgnn_aligned16(in_feat) && fgnn_aligned16(grad_out) && fgnn_aligned16(grad_feat) && fgnn_aligned16(out_feat) && fgnn_aligned16(aux_out2);
    fgnn_rowcfg cfg;
    FGNN_REQUIRE(fgnn_pick_rowcfg(HF, F, aligned, &cfg), FGNN_ERR_LIMIT, "fgnn_gat_backward: unsupported row width %d", HF);

    GatBwdP p{};
    p.items = sched_csc ? sched_csc->items_dev : nullptr;
    p.n_items = sched_csc ? sched_csc->n_items : N;
    p.ptr = col_ptr; p.idx = fgnn_sched_idx(sched_csc, row_ind); p.pos = fgnn_sched_pos(sched_csc); p.permute = permute; p.rec = rec; p.ac = attn_col; p.x = in_feat; p.g = grad_out;
    const int stash_mode = !stash ? 0 : (own_order ? 2 : 1);
    p.delta = (const float *)rec;       // own-order stash: the record area holds the compact [N,H] delta array instead
    p.esm = e_softmax; p.gfeat = grad_feat; p.gac = grad_attn_col; p.part = part;
    p.N = N; p.H = H; p.F = F; p.HF = HF; p.slope = negative_slope;

    return fgnn_dispatch_rowcfg(cfg, [&]<int VEC, int R, bool FULL>() -> int {
        float *delta_out = stash_mode == 2 ? (float *)rec : nullptr;
        if (VEC == 4 && HF <= 128 && fgnn_aligned16(out_feat) && fgnn_aligned16(aux_out2) && fgnn_aligned16(grad_out)) {
            int lpn = 1;
            while (lpn * 4 < HF) lpn *= 2;
            auto node_launch = [&]<int LPN>() {
                const int64_t waves = ((int64_t)N + 64 / LPN - 1) / (64 / LPN);
                hipLaunchKernelGGL((gat_bwd_node_packed_kernel<LPN>), dim3((unsigned)((waves + FGNN_WPB - 1) / FGNN_WPB)), dim3(FGNN_TPB), 0, st,
                                   N, H, F, HF, grad_out, out_feat, aux_out2, aux_c, attn_row, edge_max, edge_sum, rec, delta_out, grad_attn_row);
            };
            switch (lpn) {
            case 1: node_launch.template operator()<1>(); break;
            case 2: node_launch.template operator()<2>(); break;
            case 4: node_launch.template operator()<4>(); break;
            case 8: node_launch.template operator()<8>(); break;
            case 16: node_launch.template operator()<16>(); break;
            default: node_launch.template operator()<32>(); break;
            }
        } else {
            const unsigned gn = (unsigned)((N + FGNN_WPB - 1) / FGNN_WPB);
            hipLaunchKernelGGL((gat_bwd_node_kernel<VEC, R>), dim3(gn), dim3(FGNN_TPB), (size_t)FGNN_WPB * 64 * R * sizeof(float), st,
                               N, H, F, HF, grad_out, out_feat, aux_out2, aux_c, attn_row, edge_max, edge_sum, rec, delta_out, grad_attn_row);
        }
        int rc2 = fgnn_launch_status("gat_bwd_node_kernel");
        if (rc2) return rc2;
        const unsigned grid = (unsigned)((p.n_items + FGNN_WPB - 1) / FGNN_WPB);
        const size_t shm = (size_t)FGNN_WPB * (64 * R + 64) * sizeof(float);
        const bool sle1 = negative_slope >= 0.f && negative_slope <= 1.f;
        const int pack = fgnn_pick_pack(cfg.vec, HF);
        if (pack > 1) {
            p.hp_shift = 0;
            while ((1 << p.hp_shift) < H) ++p.hp_shift;
            const bool pair = ((8 * pack) << p.hp_shift) <= 64 && E >= 64 * (int64_t)N;
            const int first = sched_csc && gat_rowpack_wanted(pack, E, N) ? sched_csc->n_wave_slots : p.n_items;      // as in the forward
            const int bucketed = sched_csc && sched_csc->n_buckets > 0;
            const unsigned head_blocks = (unsigned)((first + FGNN_WPB - 1) / FGNN_WPB);
            const unsigned grid_mixed = head_blocks + fgnn_group_item_grid(p.n_items - first, pack, bucketed);
            auto launch = [&]<int G>() {
                auto go = [&]<bool PAIR>() {
                    if (first < p.n_items) {
                        if (stash_mode == 2) hipLaunchKernelGGL((gat_bwd_mixed_kernel<G, 2, true, PAIR>), dim3(grid_mixed), dim3(FGNN_TPB), shm, st, p, bucketed, first, head_blocks);
                        else if (stash_mode == 1) hipLaunchKernelGGL((gat_bwd_mixed_kernel<G, 1, true, PAIR>), dim3(grid_mixed), dim3(FGNN_TPB), shm, st, p, bucketed, first, head_blocks);
                        else if (sle1) hipLaunchKernelGGL((gat_bwd_mixed_kernel<G, 0, true, PAIR>), dim3(grid_mixed), dim3(FGNN_TPB), shm, st, p, bucketed, first, head_blocks);
                        else hipLaunchKernelGGL((gat_bwd_mixed_kernel<G, 0, false, PAIR>), dim3(grid_mixed), dim3(FGNN_TPB), shm, st, p, bucketed, first, head_blocks);
                        return;
                    }
                    if (stash_mode == 2) hipLaunchKernelGGL((gat_bwd_packed_kernel<G, 2, true, PAIR>), dim3(grid), dim3(FGNN_TPB), shm, st, p);
                    else if (stash_mode == 1) hipLaunchKernelGGL((gat_bwd_packed_kernel<G, 1, true, PAIR>), dim3(grid), dim3(FGNN_TPB), shm, st, p);
                    else if (sle1) hipLaunchKernelGGL((gat_bwd_packed_kernel<G, 0, true, PAIR>), dim3(grid), dim3(FGNN_TPB), shm, st, p);
                    else hipLaunchKernelGGL((gat_bwd_packed_kernel<G, 0, false, PAIR>), dim3(grid), dim3(FGNN_TPB), shm, st, p);
                };
                if (pair) go.template operator()<true>(); else go.template operator()<false>();
            };
            if (pack == 8) launch.template operator()<8>();
            else if (pack == 4) launch.template operator()<4>();
            else launch.template operator()<2>();
        }
        else {
            // pair layout of the attention weights, under the same conditions as in the forward
            // (7.6 -> 6.7 ms at 115 M edges, degree 492: the per-lane record reads were an L1 pass per edge)
            constexpr int U = (R >= 8) ? 1 : 8 / R;
            p.hp_shift = 0;
            while ((1 << p.hp_shift) < H) ++p.hp_shift;
            const bool pair = (U << p.hp_shift) <= 64 && E >= 64 * (int64_t)N;
            auto launch = [&]<bool PAIR>() {
                if (stash_mode == 2) hipLaunchKernelGGL((gat_bwd_kernel<VEC, R, 2, FULL, true, PAIR>), dim3(grid), dim3(FGNN_TPB), shm, st, p);
                else if (stash_mode == 1) hipLaunchKernelGGL((gat_bwd_kernel<VEC, R, 1, FULL, true, PAIR>), dim3(grid), dim3(FGNN_TPB), shm, st, p);
                else if (sle1) hipLaunchKernelGGL((gat_bwd_kernel<VEC, R, 0, FULL, true, PAIR>), dim3(grid), dim3(FGNN_TPB), shm, st, p);
                else hipLaunchKernelGGL((gat_bwd_kernel<VEC, R, 0, FULL, false, PAIR>), dim3(grid), dim3(FGNN_TPB), shm, st, p);
            };
            if (pair) launch.template operator()<true>(); else launch.template operator()<false>();
        }
        rc2 = fgnn_launch_status("gat_bwd_kernel");
        if (rc2) return rc2;
        if (sched_csc && sched_csc->n_split > 0) {
            unsigned g2 = (unsigned)((sched_csc->n_split + FGNN_WPB - 1) / FGNN_WPB);
            hipLaunchKernelGGL((gat_bwd_merge_kernel<VEC, R>), dim3(g2), dim3(FGNN_TPB), shm, st,
                               p, sched_csc->split_dev, sched_csc->n_split);
            return fgnn_launch_status("gat_bwd_merge_kernel");
        }
        return 0;
    });
}

extern "C" int fgnn_gat_backward(int N, int64_t E, int H, int F, float negative_slope, const int32_t *row_ptr,
                                 const int32_t *col_ind, const int32_t *col_ptr, const int32_t *row_ind,
                                 const int32_t *permute, const float *e_lrelu, const float *e_softmax,
                                 const float *edge_max, const float *edge_sum, const float *in_feat,
                                 const float *attn_row, const float *attn_col, const float *out_feat,
                                 const float *aux_out2, const float *aux_c, const float *grad_out, float *grad_feat,
                                 float *grad_attn_row, float *grad_attn_col, const fgnn_schedule_t *sched_csc,
                                 const fgnn_schedule_t *sched_csr, void *workspace, size_t workspace_bytes, void *stream)
{
    (void)e_lrelu;      // the sign of the pre-activation is taken from attn_row + attn_col
    return gat_backward_impl(N, E, H, F, negative_slope, row_ptr, col_ind, col_ptr, row_ind, permute, e_softmax, 0, edge_max, edge_sum, in_feat,
                             attn_row, attn_col, out_feat, aux_out2, aux_c, grad_out, grad_feat, grad_attn_row, grad_attn_col, sched_csc, sched_csr,
                             workspace, workspace_bytes, stream);
}

extern "C" int fgnn_gat_backward_own_order(int N, int64_t E, int H, int F, float negative_slope, const int32_t *row_ptr,
                                           const int32_t *col_ind, const int32_t *col_ptr, const int32_t *row_ind,
                                           const float *e_softmax_own, const float *edge_max, const float *edge_sum,
                                           const float *in_feat, const float *attn_row, const float *attn_col, const float *out_feat,
                                           const float *aux_out2, const float *aux_c, const float *grad_out, float *grad_feat,
                                           float *grad_attn_row, float *grad_attn_col, const fgnn_schedule_t *sched_csc,
                                           const fgnn_schedule_t *sched_csr, void *workspace, size_t workspace_bytes, void *stream)
{
    FGNN_REQUIRE(e_softmax_own || E == 0, FGNN_ERR_NULL, "fgnn_gat_backward_own_order: NULL stash");
    return gat_backward_impl(N, E, H, F, negative_slope, row_ptr, col_ind, col_ptr, row_ind, nullptr, e_softmax_own, e_softmax_own != nullptr, edge_max,
                             edge_sum, in_feat, attn_row, attn_col, out_feat, aux_out2, aux_c, grad_out, grad_feat, grad_attn_row, grad_attn_col,
                             sched_csc, sched_csr, workspace, workspace_bytes, stream);
}

extern "C" int fgnn_gat_stash_own_order(int N, int64_t E, int H, float negative_slope, const int32_t *col_ptr, const int32_t *row_ind,
                                        const float *attn_row, const float *attn_col, const float *edge_max, const float *edge_sum,
                                        float *e_softmax_own, const fgnn_schedule_t *sched_csc, void *stream)
{
    int rc = gat_common_checks("fgnn_gat_stash_own_order", N, E, H, 1);
    if (rc) return rc;
    FGNN_REQUIRE(col_ptr && (row_ind || E == 0) && attn_row && attn_col && edge_max && edge_sum && (e_softmax_own || E == 0), FGNN_ERR_NULL,
                 "fgnn_gat_stash_own_order: NULL argument");
    rc = check_sched(sched_csc, col_ptr, row_ind, N, E, "fgnn_gat_stash_own_order");
    if (rc) return rc;
    if (N == 0 || E == 0) return 0;
    int hp_shift = 0;
    while ((1 << hp_shift) < H) ++hp_shift;
    const int n_items = sched_csc ? sched_csc->n_items : N;
    const unsigned grid = (unsigned)((n_items + FGNN_WPB - 1) / FGNN_WPB);
    hipLaunchKernelGGL(gat_stash_own_order_kernel, dim3(grid), dim3(FGNN_TPB), 0, (hipStream_t)stream, sched_csc ? sched_csc->items_dev : nullptr,
                       n_items, col_ptr, fgnn_sched_idx(sched_csc, row_ind), H, hp_shift, attn_row, attn_col, edge_max, edge_sum, negative_slope,
                       e_softmax_own);
    return fgnn_launch_status("gat_stash_own_order_kernel");
}
