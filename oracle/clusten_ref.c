/*
 * clusten_ref.c — the CLUSTEN sums as plain C nested loops.  TEST INFRASTRUCTURE ONLY.
 *
 * A third, independent statement of what the reference kernels compute (after the PyTorch gather
 * expressions and the numpy loops in clusten_oracle.py); the tests use it to pin the gather oracle
 * on shapes that are too large for Python loops.  Inputs are float32, contiguous; every sum is
 * accumulated in double and rounded once, so its result is the correctly rounded value up to one
 * final rounding — a tighter reference than any float32 summation order.
 *
 * Index expressions follow:
 *   QK  clusten/src/clustenqk_cuda_kernel.cu:36-45 (forward), :112-129 (backward)
 *   AV  clusten/src/clustenav_cuda_kernel.cu:36-46 (forward), :110-123 (d_v), :146-156 (d_attn)
 *   WF  clusten/src/clustenwf_cuda_kernel.cu:36-50 (forward), :116-131 (d_feat), :156-165 (d_weights)
 * Nothing in the product links or loads this file.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define IDX4(a, b, c, d, B, C, D) ((((int64_t)(a) * (B) + (b)) * (C) + (c)) * (D) + (d))
#define IDX3(a, b, c, B, C) (((int64_t)(a) * (B) + (b)) * (C) + (c))

void ref_qk_forward(const float* q, const float* k, const int64_t* idx, float* attn, int b, int h, int n, int c,
                    int m) {
    for (int bi = 0; bi < b; ++bi)
        for (int hi = 0; hi < h; ++hi)
            for (int i = 0; i < n; ++i)
                for (int j = 0; j < m; ++j) {
                    const int64_t nb = idx[IDX3(bi, i, j, n, m)];
                    double s = 0.0;
                    for (int ci = 0; ci < c; ++ci)
                        s += (double)q[IDX4(bi, hi, i, ci, h, n, c)] * (double)k[IDX4(bi, hi, nb, ci, h, n, c)];
                    attn[IDX4(bi, hi, i, j, h, n, m)] = (float)s;
                }
}

void ref_av_forward(const float* attn, const float* v, const int64_t* idx, float* feat, int b, int h, int n, int c,
                    int m) {
    for (int bi = 0; bi < b; ++bi)
        for (int hi = 0; hi < h; ++hi)
            for (int i = 0; i < n; ++i)
                for (int ci = 0; ci < c; ++ci) {
                    double s = 0.0;
                    for (int j = 0; j < m; ++j) {
                        const int64_t nb = idx[IDX3(bi, i, j, n, m)];
                        s += (double)attn[IDX4(bi, hi, i, j, h, n, m)] * (double)v[IDX4(bi, hi, nb, ci, h, n, c)];
                    }
                    feat[IDX4(bi, hi, i, ci, h, n, c)] = (float)s;
                }
}

void ref_wf_forward(const float* w, const float* feat, const int64_t* idx, float* out, int b, int n, int n_out, int c,
                    int m, int ic) {
    for (int bi = 0; bi < b; ++bi)
        for (int i = 0; i < n_out; ++i)
            for (int ici = 0; ici < ic; ++ici)
                for (int ci = 0; ci < c; ++ci) {
                    double s = 0.0;
                    for (int j = 0; j < m; ++j) {
                        const int64_t nb = idx[IDX3(bi, i, j, n_out, m)];
                        s += (double)w[IDX4(bi, i, j, ici, n_out, m, ic)] * (double)feat[IDX3(bi, nb, ci, n, c)];
                    }
                    out[IDX4(bi, i, ici, ci, n_out, ic, c)] = (float)s;
                }
}

/* d_a[b,h,i,c] = sum_j rows[b,h,idx,c] * g[b,h,i,j];  d_rows[b,h,idx,c] += a[b,h,i,c] * g[b,h,i,j] */
void ref_qk_backward(const float* g, const float* q, const float* k, const int64_t* idx, float* dq, float* dk, int b,
                     int h, int n, int c, int m) {
    const int64_t total = (int64_t)b * h * n * c;
    double* dq64 = (double*)calloc((size_t)total, sizeof(double));
    double* dk64 = (double*)calloc((size_t)total, sizeof(double));
    for (int bi = 0; bi < b; ++bi)
        for (int hi = 0; hi < h; ++hi)
            for (int i = 0; i < n; ++i)
                for (int j = 0; j < m; ++j) {
                    const int64_t nb = idx[IDX3(bi, i, j, n, m)];
                    const double gij = g[IDX4(bi, hi, i, j, h, n, m)];
                    for (int ci = 0; ci < c; ++ci) {
                        dq64[IDX4(bi, hi, i, ci, h, n, c)] += (double)k[IDX4(bi, hi, nb, ci, h, n, c)] * gij;
                        dk64[IDX4(bi, hi, nb, ci, h, n, c)] += (double)q[IDX4(bi, hi, i, ci, h, n, c)] * gij;
                    }
                }
    for (int64_t t = 0; t < total; ++t) {
        dq[t] = (float)dq64[t];
        dk[t] = (float)dk64[t];
    }
    free(dq64);
    free(dk64);
}

void ref_av_backward(const float* g, const float* attn, const float* v, const int64_t* idx, float* da, float* dv,
                     int b, int h, int n, int c, int m) {
    const int64_t total_v = (int64_t)b * h * n * c;
    double* dv64 = (double*)calloc((size_t)total_v, sizeof(double));
    for (int bi = 0; bi < b; ++bi)
        for (int hi = 0; hi < h; ++hi)
            for (int i = 0; i < n; ++i)
                for (int j = 0; j < m; ++j) {
                    const int64_t nb = idx[IDX3(bi, i, j, n, m)];
                    const double aij = attn[IDX4(bi, hi, i, j, h, n, m)];
                    double s = 0.0;
                    for (int ci = 0; ci < c; ++ci) {
                        const double gic = g[IDX4(bi, hi, i, ci, h, n, c)];
                        s += (double)v[IDX4(bi, hi, nb, ci, h, n, c)] * gic;
                        dv64[IDX4(bi, hi, nb, ci, h, n, c)] += aij * gic;
                    }
                    da[IDX4(bi, hi, i, j, h, n, m)] = (float)s;
                }
    for (int64_t t = 0; t < total_v; ++t) dv[t] = (float)dv64[t];
    free(dv64);
}

void ref_wf_backward(const float* g, const float* w, const float* feat, const int64_t* idx, float* dw, float* df,
                     int b, int n, int n_out, int c, int m, int ic) {
    const int64_t total_f = (int64_t)b * n * c;
    double* df64 = (double*)calloc((size_t)total_f, sizeof(double));
    for (int bi = 0; bi < b; ++bi)
        for (int i = 0; i < n_out; ++i)
            for (int j = 0; j < m; ++j) {
                const int64_t nb = idx[IDX3(bi, i, j, n_out, m)];
                for (int ici = 0; ici < ic; ++ici) {
                    const double wij = w[IDX4(bi, i, j, ici, n_out, m, ic)];
                    double s = 0.0;
                    for (int ci = 0; ci < c; ++ci) {
                        const double gc = g[IDX4(bi, i, ici, ci, n_out, ic, c)];
                        s += (double)feat[IDX3(bi, nb, ci, n, c)] * gc;
                        df64[IDX3(bi, nb, ci, n, c)] += gc * wij;
                    }
                    dw[IDX4(bi, i, j, ici, n_out, m, ic)] = (float)s;
                }
            }
    for (int64_t t = 0; t < total_f; ++t) df[t] = (float)df64[t];
    free(df64);
}
