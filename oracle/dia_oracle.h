/*
 * dia_oracle.h -- CPU restatement of CUV's host_memory_space DIA path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product (the HIP library, the
 * cuv_amd package, the C++ mirror headers) may include, link or call this
 * file; it exists so that tests, the smoke check and the bench's CPU
 * baseline leg have something independent to compare the GPU against.
 *
 * Every function restates, loop for loop, one function of the reference
 * (paths relative to the reference checkout):
 *
 *   oracle_spmv_f32            src/cuv/matrix_ops/spmv.cu:145-200
 *   oracle_prod_dia_f32        src/cuv/matrix_ops/spmv.cu:203-220
 *   oracle_dd2dia_literal_f32  src/cuv/matrix_ops/densedense_to_sparse.cu:204-252
 *   oracle_dd2dia_f32          same loop order, with the documented
 *                              C = factC*C + factAB*A*B' contract of
 *                              densedense_to_sparse.hpp:107-121 and the
 *                              store of densedense_to_sparse.cu:110-111
 *   oracle_dia_get_f32         src/cuv/basics/dia_matrix.hpp:236-243
 *   oracle_dia_to_dense_f32    src/cuv/convert/convert.cu:42-66
 *   oracle_filter_offsets      src/cuv/basics/filter_factory.hpp:43-76
 *   oracle_avg_diagonals_f32   src/cuv/matrix_ops/diagonals.cu:24-51
 *
 * The *_f64 variants run the same loops with double accumulators and are
 * used to budget rounding error; the *_mag variants return sum |term| per
 * output, the scale a mixed tolerance is expressed against.
 *
 * Build with -ffp-contract=off: the reference computes mul, mul, add with
 * a rounding after each (spmv.cu:176,196); a fused multiply-add would
 * change the bits.
 *
 * Pinning status (what checks each function without running the reference):
 *   spmv / prod_dia        closed forms of src/tests/spmv.cpp:65-143 (exact
 *                          integers in fp32), dense fp64 GEMV cross-check,
 *                          transpose identity, brute force for rf in {1,2,4}
 *   dd2dia_literal         closed form of src/tests/densedense_to_dia.cpp:
 *                          66-137 (rf=4), brute-force projection of A*B'
 *   dd2dia (alpha,beta)    PARITY UNPINNED against the reference host code:
 *                          the host loop never reads factAB/factC; only the
 *                          documented contract and the device kernel's
 *                          store expression define it.  Pinned against the
 *                          mathematics (linearity in alpha, beta=0 ignores
 *                          dst, alpha=beta=1 equals the literal loop).
 *   dia_get / dia_to_dense closed form of src/tests/dia_mat.cpp:65-119 and
 *                          src/tests/convert.cpp:110-129
 *   filter_offsets         closed form (arithmetic progression per window row)
 *   avg_diagonals          mean of the closed-form sequence() diagonals
 */
#ifndef DIA_ORACLE_H
#define DIA_ORACLE_H

#ifdef __cplusplus
extern "C" {
#endif

/* y (len h for 'n', w for 't') = factC*y + factAv*op(A)*x.  Returns 0, or
 * -1 if transA is neither 'n' nor 't'. */
int oracle_spmv_f32(int h, int w, int nd, int stride, int rf,
                    const int *offsets, const float *A_vals,
                    const float *x, float *y,
                    char transA, float factAv, float factC);

/* Column loop over a column-major batch: dst[:,c] <- spmv(B[:,c]).
 * B is n_in x batch with leading dimension n_in, dst n_out x batch with
 * leading dimension n_out (the reference takes both from shape[0]). */
int oracle_prod_dia_f32(int h, int w, int nd, int stride, int rf,
                        const int *offsets, const float *A_vals,
                        const float *B, float *dst, int batch,
                        char transA, float factAB, float factC);

/* Same contraction, double accumulators, result in double:
 * out = factC*dst_in + factAB*op(A)*B  (dst_in may be NULL when factC==0). */
int oracle_prod_dia_f64(int h, int w, int nd, int stride, int rf,
                        const int *offsets, const float *A_vals,
                        const float *B, const float *dst_in, double *out,
                        int batch, char transA, float factAB, float factC);

/* mag = |factC*dst_in| + sum_d |factAB*a*x| per output element. */
int oracle_prod_dia_mag(int h, int w, int nd, int stride, int rf,
                        const int *offsets, const float *A_vals,
                        const float *B, const float *dst_in, double *mag,
                        int batch, char transA, float factAB, float factC);

/* Literal host loop: C_d[row] += A[row,c]*B[col,c], diagonal by diagonal,
 * column by column; factAB and factC do not appear (as in the reference).
 * Returns -2 if some diagonal's N is not a multiple of rf (the reference
 * loop over-runs its end pointer there: undefined). */
int oracle_dd2dia_literal_f32(int h, int w, int nd, int stride, int rf,
                              const int *offsets, float *C_vals,
                              const float *A, const float *B, int batch);

/* Documented contract in the literal loop's order: S accumulated from 0
 * over columns c = 0..batch-1, then C = factC*C + factAB*S (factC==0 never
 * reads C). */
int oracle_dd2dia_f32(int h, int w, int nd, int stride, int rf,
                      const int *offsets, float *C_vals,
                      const float *A, const float *B, int batch,
                      float factAB, float factC);

/* Double-accumulator shadow; out has the layout of C_vals (nd*stride);
 * slots no diagonal element maps to are copied from C_in (or 0). */
int oracle_dd2dia_f64(int h, int w, int nd, int stride, int rf,
                      const int *offsets, const float *C_in, double *out,
                      const float *A, const float *B, int batch,
                      float factAB, float factC);

/* Element (i,j): offset j - i/rf looked up in the table; the LAST table
 * entry with that offset wins (std::map overwrite in post_update_offsets,
 * dia_matrix.hpp:181-185); 0 when the offset is not stored. */
float oracle_dia_get_f32(int h, int w, int nd, int stride, int rf,
                         const int *offsets, const float *A_vals,
                         int i, int j);

/* dense is h x w column-major (ld = h); zero-filled first. */
int oracle_dia_to_dense_f32(int h, int w, int nd, int stride, int rf,
                            const int *offsets, const float *A_vals,
                            float *dense);

/* Offsets of a locally connected layer: fs x fs window on a px x py map,
 * input_maps -> output_maps.  Writes fs*fs*(output_maps+input_maps-1)
 * ints and returns that count. */
int oracle_filter_offsets(int px, int py, int fs, int input_maps,
                          int output_maps, int *offsets_out);

/* Mean over the valid part of each stored diagonal (host variant). */
int oracle_avg_diagonals_f32(int h, int w, int nd, int stride,
                             const int *offsets, const float *A_vals,
                             float *avg_out);

#ifdef __cplusplus
}
#endif
#endif
