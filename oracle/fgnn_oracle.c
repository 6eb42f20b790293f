/*
 * CPU oracle in plain C for the fused GNN sparse-operator path.
 *
 * TEST INFRASTRUCTURE ONLY: this file is the checker.  It is compiled into
 * oracle/_build/libfgnn_oracle.so and loaded by tests, the smoke entry and the
 * CPU-baseline leg of the benchmark.  The shipped library never links, loads or
 * calls it.
 *
 * Every routine is an explicit loop nest over CSR rows (row = destination node,
 * col_ind = source node, per-edge arrays in CSR position order) in double
 * precision.  It is written independently of the torch restatement in
 * fgnn_oracle.py (segment ops + autograd) so that the two pin each other: the
 * backward routines here are the analytic formulas, the torch side differentiates
 * the forward numerically exact through autograd.
 *
 * Reference lines each routine follows are cited at the routine.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static double lrelu(double x, double slope) { return x > 0.0 ? x : slope * x; }

/* GAT forward.  Math of src/fused_gat/fused_gat_SM.cu:193-286 (three passes per row and
 * head: max, sum of exp, weighted accumulation) == GATConv_dgl.forward
 * (layers/gatconv_layer.py:204-210).  Empty rows: out = 0, edge_max = -1e38, edge_sum = 0. */
void fgo_gat_forward(int n, int h, int f, const int32_t *row_ptr, const int32_t *col_ind,
                     const double *attn_row, const double *attn_col, double slope,
                     const double *in_feat, double *out, double *edge_max, double *edge_sum)
{
    for (int i = 0; i < n; ++i) {
        for (int hh = 0; hh < h; ++hh) {
            double m = -1e38, s = 0.0;
            for (int p = row_ptr[i]; p < row_ptr[i + 1]; ++p) {
                double e = lrelu(attn_row[(size_t)i * h + hh] + attn_col[(size_t)col_ind[p] * h + hh], slope);
                if (e > m) m = e;
            }
            for (int p = row_ptr[i]; p < row_ptr[i + 1]; ++p) {
                double e = lrelu(attn_row[(size_t)i * h + hh] + attn_col[(size_t)col_ind[p] * h + hh], slope);
                s += exp(e - m);
            }
            double *o = out + ((size_t)i * h + hh) * f;
            for (int k = 0; k < f; ++k) o[k] = 0.0;
            for (int p = row_ptr[i]; p < row_ptr[i + 1]; ++p) {
                int j = col_ind[p];
                double e = lrelu(attn_row[(size_t)i * h + hh] + attn_col[(size_t)j * h + hh], slope);
                double a = exp(e - m) / s;
                const double *x = in_feat + ((size_t)j * h + hh) * f;
                for (int k = 0; k < f; ++k) o[k] += a * x[k];
            }
            edge_max[(size_t)i * h + hh] = m;
            edge_sum[(size_t)i * h + hh] = s;
        }
    }
}

/* GAT backward, analytic.  Follows src/fused_gat/fused_gat_SM.cu:560-607 (grad_feat by
 * alpha-weighted sum of grad rows), :656-732 (per-edge dot products), :734-801 (softmax and
 * LeakyReLU backward).  The derivative of LeakyReLU at exactly 0 is `slope`, as in
 * torch.nn.functional.leaky_relu (the reference kernel uses 1 there; exact zeros are kept
 * out of gradient fixtures).  Works from CSR only: the scatter into source nodes is done
 * with plain += on the CPU. */
void fgo_gat_backward(int n, int h, int f, const int32_t *row_ptr, const int32_t *col_ind,
                      const double *attn_row, const double *attn_col, double slope,
                      const double *in_feat, const double *grad_out, double *grad_feat,
                      double *grad_attn_row, double *grad_attn_col)
{
    memset(grad_feat, 0, sizeof(double) * (size_t)n * h * f);
    memset(grad_attn_row, 0, sizeof(double) * (size_t)n * h);
    memset(grad_attn_col, 0, sizeof(double) * (size_t)n * h);
    for (int i = 0; i < n; ++i) {
        int b = row_ptr[i], e_ = row_ptr[i + 1];
        if (b == e_) continue;
        for (int hh = 0; hh < h; ++hh) {
            double m = -1e38, s = 0.0;
            for (int p = b; p < e_; ++p) {
                double e = lrelu(attn_row[(size_t)i * h + hh] + attn_col[(size_t)col_ind[p] * h + hh], slope);
                if (e > m) m = e;
            }
            for (int p = b; p < e_; ++p) {
                double e = lrelu(attn_row[(size_t)i * h + hh] + attn_col[(size_t)col_ind[p] * h + hh], slope);
                s += exp(e - m);
            }
            const double *g = grad_out + ((size_t)i * h + hh) * f;
            /* ws = sum_p alpha_p * ge_p */
            double ws = 0.0;
            for (int p = b; p < e_; ++p) {
                int j = col_ind[p];
                double e = lrelu(attn_row[(size_t)i * h + hh] + attn_col[(size_t)j * h + hh], slope);
                double a = exp(e - m) / s;
                const double *x = in_feat + ((size_t)j * h + hh) * f;
                double ge = 0.0;
                for (int k = 0; k < f; ++k) ge += g[k] * x[k];
                ws += a * ge;
            }
            for (int p = b; p < e_; ++p) {
                int j = col_ind[p];
                double e = lrelu(attn_row[(size_t)i * h + hh] + attn_col[(size_t)j * h + hh], slope);
                double a = exp(e - m) / s;
                const double *x = in_feat + ((size_t)j * h + hh) * f;
                double *gx = grad_feat + ((size_t)j * h + hh) * f;
                double ge = 0.0;
                for (int k = 0; k < f; ++k) { ge += g[k] * x[k]; gx[k] += a * g[k]; }
                double gg = a * (ge - ws) * (e > 0.0 ? 1.0 : slope);
                grad_attn_row[(size_t)i * h + hh] += gg;
                grad_attn_col[(size_t)j * h + hh] += gg;
            }
        }
    }
}

/* EdgeConv forward.  Contract of operators/fused_edgeconv.py:18-29 with the tie rule of the
 * DGL max reducer that layers/edgeconv_layer.py:102-109 uses: the first maximal CSR position
 * wins (strict > update).  Values are single precision because the result must be the
 * bit-exact fp32 sum h_dst + h_src of the winning candidate. */
void fgo_edgeconv_forward(int n, int f, int k, const int32_t *src_ind, const float *h_src,
                          const float *h_dst, float *out, int32_t *argmax)
{
    for (int i = 0; i < n; ++i)
        for (int c = 0; c < f; ++c) {
            float best = 0.0f; int32_t arg = -1;
            for (int t = 0; t < k; ++t) {
                int j = src_ind[(size_t)i * k + t];
                float v = h_dst[(size_t)i * f + c] + h_src[(size_t)j * f + c];
                if (t == 0 || v > best) { best = v; arg = j; }
            }
            out[(size_t)i * f + c] = best;
            argmax[(size_t)i * f + c] = arg;
        }
}

/* EdgeConv backward: grad_src[argmax[i,c], c] += grad_out[i,c]
 * (src/fused_edgeconv/fused_edgeconv.cu:175-187 without its zero-vs-atomic race). */
void fgo_edgeconv_backward(int n, int n_src, int f, const int32_t *argmax, const double *grad_out,
                           double *grad_src)
{
    memset(grad_src, 0, sizeof(double) * (size_t)n_src * f);
    for (int i = 0; i < n; ++i)
        for (int c = 0; c < f; ++c)
            grad_src[(size_t)argmax[(size_t)i * f + c] * f + c] += grad_out[(size_t)i * f + c];
}

/* Gaussian mixture weights, src/fused_gmmconv/gmmconv.cu:34-45 (intended math; also
 * layers/gmmconv_layer.py:136-139). */
static double gauss_w(const double *ps, const double *mu, const double *isg, int dim)
{
    double acc = 0.0;
    for (int d = 0; d < dim; ++d) { double t = (ps[d] - mu[d]) * isg[d]; acc += t * t; }
    return exp(-0.5 * acc);
}

/* GMMConv forward, src/fused_gmmconv/gmmconv.cu:48-80 (intended math, without its shared
 * memory index overlap) == layers/gmmconv_layer.py:140-142. */
void fgo_gmm_forward(int n, int kk, int dim, int f, const int32_t *row_ptr, const int32_t *col_ind,
                     const double *node_feat, const double *pseudo, const double *mu,
                     const double *inv_sigma, double *out)
{
    memset(out, 0, sizeof(double) * (size_t)n * kk * f);
    for (int i = 0; i < n; ++i)
        for (int p = row_ptr[i]; p < row_ptr[i + 1]; ++p) {
            int j = col_ind[p];
            for (int k = 0; k < kk; ++k) {
                double w = gauss_w(pseudo + (size_t)p * dim, mu + (size_t)k * dim, inv_sigma + (size_t)k * dim, dim);
                const double *x = node_feat + ((size_t)j * kk + k) * f;
                double *o = out + ((size_t)i * kk + k) * f;
                for (int c = 0; c < f; ++c) o[c] += w * x[c];
            }
        }
}

/* GMMConv backward, closed forms (the operator sequence of operators/fused_gmmconv.py:51-58;
 * the reference's gaussian_bp kernel, gmmconv.cu:154-184, does not compute these and is not
 * followed).  d/dmu = gw*w*(p-mu)*isg^2, d/disg = -gw*w*(p-mu)^2*isg, d/dp = -gw*w*(p-mu)*isg^2. */
void fgo_gmm_backward(int n, int kk, int dim, int f, const int32_t *row_ptr, const int32_t *col_ind,
                      const double *node_feat, const double *pseudo, const double *mu,
                      const double *inv_sigma, const double *grad_out, double *grad_feat,
                      double *grad_pseudo, double *grad_mu, double *grad_sigma)
{
    size_t ne = (size_t)row_ptr[n];
    memset(grad_feat, 0, sizeof(double) * (size_t)n * kk * f);
    memset(grad_pseudo, 0, sizeof(double) * ne * dim);
    memset(grad_mu, 0, sizeof(double) * (size_t)kk * dim);
    memset(grad_sigma, 0, sizeof(double) * (size_t)kk * dim);
    for (int i = 0; i < n; ++i)
        for (int p = row_ptr[i]; p < row_ptr[i + 1]; ++p) {
            int j = col_ind[p];
            for (int k = 0; k < kk; ++k) {
                const double *ps = pseudo + (size_t)p * dim;
                const double *m = mu + (size_t)k * dim, *sg = inv_sigma + (size_t)k * dim;
                double w = gauss_w(ps, m, sg, dim);
                const double *x = node_feat + ((size_t)j * kk + k) * f;
                const double *g = grad_out + ((size_t)i * kk + k) * f;
                double *gx = grad_feat + ((size_t)j * kk + k) * f;
                double gw = 0.0;
                for (int c = 0; c < f; ++c) { gw += g[c] * x[c]; gx[c] += w * g[c]; }
                for (int d = 0; d < dim; ++d) {
                    double diff = ps[d] - m[d];
                    grad_mu[(size_t)k * dim + d] += gw * w * diff * sg[d] * sg[d];
                    grad_sigma[(size_t)k * dim + d] -= gw * w * diff * diff * sg[d];
                    grad_pseudo[(size_t)p * dim + d] -= gw * w * diff * sg[d] * sg[d];
                }
            }
        }
}

/* Stable CSR -> CSC transpose by counting sort; what the reference scripts obtain from scipy
 * (script/train/train_gmmconv_our.py:80-93).  permute[q] = CSR position of CSC entry q. */
void fgo_csr2csc(int n_rows, int n_cols, const int32_t *row_ptr, const int32_t *col_ind,
                 int32_t *col_ptr, int32_t *row_ind, int32_t *permute)
{
    int32_t *next = (int32_t *)calloc((size_t)n_cols + 1, sizeof(int32_t));
    for (int p = 0; p < row_ptr[n_rows]; ++p) next[col_ind[p] + 1]++;
    col_ptr[0] = 0;
    for (int c = 0; c < n_cols; ++c) { next[c + 1] += next[c]; col_ptr[c + 1] = next[c + 1]; }
    for (int i = 0; i < n_rows; ++i)
        for (int p = row_ptr[i]; p < row_ptr[i + 1]; ++p) {
            int q = next[col_ind[p]]++;
            row_ind[q] = i;
            permute[q] = p;
        }
    free(next);
}
