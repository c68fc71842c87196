/*
 * dia_oracle.c -- CPU restatement of CUV's host_memory_space DIA path.
 *
 * TEST INFRASTRUCTURE ONLY (see dia_oracle.h).  Compile with
 * -O2 -ffp-contract=off so that every multiply and add rounds on its own,
 * as the reference's scalar loops do.
 *
 * One deliberate difference from the reference: its index type is
 * `unsigned int`, so a diagonal whose offset lies outside the matrix makes
 * `A_w - j_start` wrap and the loop read out of bounds (undefined).  Here
 * the counts are signed and such a diagonal contributes nothing.
 */
#include "dia_oracle.h"

#include <stdlib.h>
#include <string.h>
#include <math.h>

static int imax(int a, int b) { return a > b ? a : b; }
static int imin(int a, int b) { return a < b ? a : b; }

/* ---- spmv: src/cuv/matrix_ops/spmv.cu:145-200 --------------------------- */
int oracle_spmv_f32(int h, int w, int nd, int stride, int rf,
                    const int *offsets, const float *A_vals,
                    const float *x, float *y,
                    char transA, float factAv, float factC)
{
    if (transA != 'n' && transA != 't') return -1;
    const int max_dst = (transA == 't') ? w : h;
    /* spmv.cu:152-156: zero-fill when factC == 0 (dst is never read) */
    if (factC == 0.f)
        for (int i = 0; i < max_dst; i++) y[i] = 0.f;
    else
        for (int i = 0; i < max_dst; i++) y[i] = y[i] * factC;

    if (transA == 't') {
        /* spmv.cu:158-178 */
        for (int d = 0; d < nd; d++) {
            const int k = offsets[d];
            const int i_start = imax(0, k);
            const int j_start = rf * imax(0, -k);
            const int N = imin((h - j_start) / rf, w - i_start);
            const float *d_ = A_vals + (size_t)d * stride + j_start;
            const float *x_ = x + j_start;
            float *y_ = y + i_start;
            for (int n = 0; n < N; n++, y_++)
                for (int q = 0; q < rf; q++, x_++, d_++)
                    *y_ += factAv * *d_ * *x_;
        }
    } else {
        /* spmv.cu:179-199 */
        for (int d = 0; d < nd; d++) {
            const int k = offsets[d];
            const int i_start = rf * imax(0, -k);
            const int j_start = imax(0, k);
            const int N = imin(h - i_start, rf * (w - j_start));
            const float *d_ = A_vals + (size_t)d * stride + i_start;
            const float *x_ = x + j_start;
            float *y_ = y + i_start;
            for (int n = 0; n < N; n++)
                *y_++ += factAv * *d_++ * x_[n / rf];
        }
    }
    return 0;
}

/* ---- prod(dst, dia, dense): src/cuv/matrix_ops/spmv.cu:203-220 ---------- */
int oracle_prod_dia_f32(int h, int w, int nd, int stride, int rf,
                        const int *offsets, const float *A_vals,
                        const float *B, float *dst, int batch,
                        char transA, float factAB, float factC)
{
    if (transA != 'n' && transA != 't') return -1;
    const size_t n_out = (transA == 't') ? w : h;
    const size_t n_in  = (transA == 't') ? h : w;
    for (int c = 0; c < batch; c++) {
        int rc = oracle_spmv_f32(h, w, nd, stride, rf, offsets, A_vals,
                                 B + c * n_in, dst + c * n_out,
                                 transA, factAB, factC);
        if (rc) return rc;
    }
    return 0;
}

/* Walk the same (d, n, q) index space once, handing every term to `fn`. */
typedef void (*term_fn)(void *ctx, size_t out_idx, float a, float x);

static void walk_terms(int h, int w, int nd, int stride, int rf,
                       const int *offsets, const float *A_vals,
                       const float *x, char transA, term_fn fn, void *ctx)
{
    if (transA == 't') {
        for (int d = 0; d < nd; d++) {
            const int k = offsets[d];
            const int i_start = imax(0, k);
            const int j_start = rf * imax(0, -k);
            const int N = imin((h - j_start) / rf, w - i_start);
            for (int n = 0; n < N; n++)
                for (int q = 0; q < rf; q++) {
                    const int r = j_start + n * rf + q;
                    fn(ctx, (size_t)(i_start + n),
                       A_vals[(size_t)d * stride + r], x[r]);
                }
        }
    } else {
        for (int d = 0; d < nd; d++) {
            const int k = offsets[d];
            const int i_start = rf * imax(0, -k);
            const int j_start = imax(0, k);
            const int N = imin(h - i_start, rf * (w - j_start));
            for (int n = 0; n < N; n++)
                fn(ctx, (size_t)(i_start + n),
                   A_vals[(size_t)d * stride + i_start + n],
                   x[j_start + n / rf]);
        }
    }
}

struct acc_ctx { double *out; double f; };
static void acc_term(void *c, size_t o, float a, float x)
{
    struct acc_ctx *k = (struct acc_ctx *)c;
    k->out[o] += k->f * (double)a * (double)x;
}
static void mag_term(void *c, size_t o, float a, float x)
{
    struct acc_ctx *k = (struct acc_ctx *)c;
    k->out[o] += fabs(k->f * (double)a * (double)x);
}

static int prod_shadow(int h, int w, int nd, int stride, int rf,
                       const int *offsets, const float *A_vals,
                       const float *B, const float *dst_in, double *out,
                       int batch, char transA, float factAB, float factC,
                       int want_mag)
{
    if (transA != 'n' && transA != 't') return -1;
    const size_t n_out = (transA == 't') ? w : h;
    const size_t n_in  = (transA == 't') ? h : w;
    for (int c = 0; c < batch; c++) {
        double *o = out + c * n_out;
        for (size_t i = 0; i < n_out; i++) {
            double v = (factC == 0.f || !dst_in)
                           ? 0.0 : (double)factC * (double)dst_in[c * n_out + i];
            o[i] = want_mag ? fabs(v) : v;
        }
        struct acc_ctx ctx = { o, (double)factAB };
        walk_terms(h, w, nd, stride, rf, offsets, A_vals, B + c * n_in,
                   transA, want_mag ? mag_term : acc_term, &ctx);
    }
    return 0;
}

int oracle_prod_dia_f64(int h, int w, int nd, int stride, int rf,
                        const int *offsets, const float *A_vals,
                        const float *B, const float *dst_in, double *out,
                        int batch, char transA, float factAB, float factC)
{
    return prod_shadow(h, w, nd, stride, rf, offsets, A_vals, B, dst_in, out,
                       batch, transA, factAB, factC, 0);
}

int oracle_prod_dia_mag(int h, int w, int nd, int stride, int rf,
                        const int *offsets, const float *A_vals,
                        const float *B, const float *dst_in, double *mag,
                        int batch, char transA, float factAB, float factC)
{
    return prod_shadow(h, w, nd, stride, rf, offsets, A_vals, B, dst_in, mag,
                       batch, transA, factAB, factC, 1);
}

/* ---- densedense_to_dia host: densedense_to_sparse.cu:204-252 ------------ */
int oracle_dd2dia_literal_f32(int h, int w, int nd, int stride, int rf,
                              const int *offsets, float *C_vals,
                              const float *A, const float *B, int batch)
{
    const size_t Ah = h, Bh = w;
    float *dst_diabase = C_vals;
    for (int dia = 0; dia < nd; dia++, dst_diabase += stride) {
        const int k = offsets[dia];
        const int row_start = rf * imax(0, -k);
        const int col_start = imax(0, k);
        const int N = imin(h - row_start, rf * (w - col_start));
        if (N <= 0) continue;
        if (N % rf) return -2;
        float *const d_base = dst_diabase + row_start;
        const float *a = A + row_start;
        const float *b = B + col_start;
        const float *const a_end = a + (size_t)batch * Ah;
        float *const d_end = d_base + N;
        for (; a < a_end; a += Ah, b += Bh) {
            float *d = d_base;
            while (d < d_end) {
                for (int q = 1; q < rf; q++)
                    *d++ += (*a++) * (*b);
                *d++ += (*a++) * (*b++);
            }
            a -= N; b -= N / rf;
        }
    }
    return 0;
}

int oracle_dd2dia_f32(int h, int w, int nd, int stride, int rf,
                      const int *offsets, float *C_vals,
                      const float *A, const float *B, int batch,
                      float factAB, float factC)
{
    const size_t Ah = h, Bh = w;
    float *S = (float *)malloc(sizeof(float) * (size_t)imax(h, 1));
    if (!S) return -3;
    for (int dia = 0; dia < nd; dia++) {
        const int k = offsets[dia];
        const int row_start = rf * imax(0, -k);
        const int col_start = imax(0, k);
        const int N = imin(h - row_start, rf * (w - col_start));
        if (N <= 0) continue;
        for (int n = 0; n < N; n++) S[n] = 0.f;
        /* same sweep as the literal loop: column by column, then along n */
        for (int c = 0; c < batch; c++) {
            const float *a = A + c * Ah + row_start;
            const float *b = B + c * Bh + col_start;
            for (int n = 0; n < N; n++)
                S[n] += a[n] * b[n / rf];
        }
        float *d = C_vals + (size_t)dia * stride + row_start;
        /* densedense_to_sparse.cu:110-118: factC*C + factAB*Csub, and no
         * read of C when factC == 0 */
        if (factC == 0.f)
            for (int n = 0; n < N; n++) d[n] = factAB * S[n];
        else
            for (int n = 0; n < N; n++) d[n] = factC * d[n] + factAB * S[n];
    }
    free(S);
    return 0;
}

int oracle_dd2dia_f64(int h, int w, int nd, int stride, int rf,
                      const int *offsets, const float *C_in, double *out,
                      const float *A, const float *B, int batch,
                      float factAB, float factC)
{
    const size_t Ah = h, Bh = w;
    const size_t total = (size_t)nd * stride;
    for (size_t i = 0; i < total; i++) out[i] = C_in ? (double)C_in[i] : 0.0;
    for (int dia = 0; dia < nd; dia++) {
        const int k = offsets[dia];
        const int row_start = rf * imax(0, -k);
        const int col_start = imax(0, k);
        const int N = imin(h - row_start, rf * (w - col_start));
        for (int n = 0; n < N; n++) {
            double s = 0.0;
            for (int c = 0; c < batch; c++)
                s += (double)A[c * Ah + row_start + n] *
                     (double)B[c * Bh + col_start + n / rf];
            const size_t idx = (size_t)dia * stride + row_start + n;
            const double old = (factC == 0.f || !C_in)
                                   ? 0.0 : (double)factC * (double)C_in[idx];
            out[idx] = old + (double)factAB * s;
        }
    }
    return 0;
}

/* ---- element access: src/cuv/basics/dia_matrix.hpp:236-243 -------------- */
float oracle_dia_get_f32(int h, int w, int nd, int stride, int rf,
                         const int *offsets, const float *A_vals,
                         int i, int j)
{
    (void)h; (void)w;
    const int off = j - i / rf;
    int found = -1;
    for (int d = 0; d < nd; d++)           /* last entry wins, like the map */
        if (offsets[d] == off) found = d;
    if (found < 0) return 0.f;
    return A_vals[(size_t)found * stride + i];
}

/* ---- dia -> dense: src/cuv/convert/convert.cu:42-66 --------------------- */
int oracle_dia_to_dense_f32(int h, int w, int nd, int stride, int rf,
                            const int *offsets, const float *A_vals,
                            float *dense)
{
    memset(dense, 0, sizeof(float) * (size_t)h * w);
    for (int oi = 0; oi < nd; oi++) {
        const int o = offsets[oi];
        int j = imax(0, o);
        int i = rf * imax(0, -o);
        for (; i < h && j < w; j++)
            for (int q = 0; q < rf; q++, i++) {
                if (i >= h) break;          /* guard the reference lacks */
                dense[(size_t)j * h + i] =
                    oracle_dia_get_f32(h, w, nd, stride, rf, offsets, A_vals, i, j);
            }
    }
    return 0;
}

/* ---- filter_factory::get_dia offsets: filter_factory.hpp:43-76 ---------- */
int oracle_filter_offsets(int px, int py, int fs, int input_maps,
                          int output_maps, int *off)
{
    const int nm = output_maps;
    const int msize = fs * fs * (nm + input_maps - 1);
    int idx = 0;
    for (int m = 0; m < nm + input_maps - 1; m++)
        for (int i = 0; i < fs; i++)
            for (int j = 0; j < fs; j++)
                off[idx++] = i * px + j + m * px * py;
    for (int i = 0; i < msize; i++)
        off[i] += -(px + 1) * (fs / 2) - (input_maps - 1) * px * py;
    return msize;
}

/* ---- avg_diagonals host: src/cuv/matrix_ops/diagonals.cu:24-51 ---------- */
int oracle_avg_diagonals_f32(int h, int w, int nd, int stride,
                             const int *offsets, const float *A_vals,
                             float *avg_out)
{
    for (int i = 0; i < nd; i++) {
        float sum = 0.f;
        const int k = offsets[i];
        const int i_start = imax(0, -k);
        const int j_start = imax(0, k);
        const int N = imin(h - i_start, w - j_start);
        const float *d = A_vals + (size_t)i * stride + i_start;
        for (int j = 0; j < N; j++) sum += *d++;
        avg_out[i] = sum / (float)N;
    }
    return 0;
}
