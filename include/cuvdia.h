/*
 * cuvdia.h -- C ABI of the MI355X (gfx950) diagonal-sparse product library.
 *
 * This is the drop-in boundary for CUV's DIA matrix path: the entry points
 * below are what the dev_memory_space specialisations of cuv::prod /
 * cuv::spmv / cuv::densedense_to_dia bind instead of launching the CUDA
 * kernels.  Reference files are cited relative to the CUV checkout.
 *
 * Conventions
 *   - plain pointers and sizes only; every float/int buffer named "device"
 *     is a raw hipMalloc pointer on the current device; "host" buffers are
 *     ordinary host memory;
 *   - dense operands are fp32, column-major, with an explicit leading
 *     dimension in elements (the reference always uses ld == rows,
 *     src/cuv/matrix_ops/spmv.cu:243-244);
 *   - a DIA matrix stores element (i, j) at vals[d*stride + i] where
 *     offsets[d] == j - i/row_fact (src/cuv/basics/dia_matrix.hpp:228-243);
 *     slots of a stored diagonal that map to no matrix element (padding) are
 *     never read and never written;
 *   - every call returns CUVDIA_OK (0) or a negative CUVDIA_E* code and
 *     never throws; kernels are enqueued on `stream` (a hipStream_t passed
 *     as void*, NULL = the default stream) and the call returns without
 *     synchronising -- the C++ mirror synchronises to keep the reference's
 *     "results visible on return" behaviour (spmv.cu:99,
 *     densedense_to_sparse.cu:295);
 *   - no entry point allocates device memory except cuvdia_desc_create and
 *     the first use of a new offset table by the *_offsets_* forms
 *     (cuvdia_spmm_offsets_noalloc_f32 never does);
 *   - a descriptor belongs to the device that was current when it was
 *     created; a compute call made while another device is current returns
 *     CUVDIA_EINVAL.  The *_offsets_* forms keep one descriptor per device.
 */
#ifndef CUVDIA_H
#define CUVDIA_H

#ifdef __cplusplus
extern "C" {
#endif

#define CUVDIA_OK            0
#define CUVDIA_EINVAL       -1  /* null pointer, bad flag, non-positive size     */
#define CUVDIA_ESHAPE       -2  /* operand shapes inconsistent with the matrix    */
#define CUVDIA_EHIP         -3  /* a HIP runtime call failed                      */
#define CUVDIA_ENOMEM       -4  /* host or device allocation failed               */
#define CUVDIA_EUNSUPPORTED -5  /* valid request this build has no kernel for     */
#define CUVDIA_ENODEVICE    -6  /* no gfx950 device visible                       */
#define CUVDIA_ETOOLARGE    -7  /* beyond the fixed capacity of cuvdia_spmm_offsets_noalloc_f32 */

/* Kernel families, for cuvdia_set_path / cuvdia_last_path. */
#define CUVDIA_PATH_AUTO     0  /* pick by shape (default)                        */
#define CUVDIA_PATH_GENERIC  1  /* one-thread-per-output kernels, any row_fact    */
#define CUVDIA_PATH_TILED    2  /* LDS-staged, register-blocked kernels (rf == 1) */
#define CUVDIA_PATH_WALK     3  /* of the tiled family: the walking kernel for window tables (products only) */
#define CUVDIA_PATH_TILED_NOWALK 4  /* the tiled family without its kernels for window tables                  */
#define CUVDIA_PATH_WINDOW   5  /* of the tiled family: the projection tiled in the window's plane (window tables) */

/* Activation applied by cuvdia_spmm_bias_act_f32. */
#define CUVDIA_ACT_NONE      0
#define CUVDIA_ACT_SIGMOID   1  /* 1 / (1 + exp(-x)), src/cuv/tensor_ops/functors.hpp:122 */
#define CUVDIA_ACT_SIGMOID_SAMPLE 2  /* the sigmoid, then a Bernoulli sample of it (cuvdia_spmm_layer_f32 only) */

/* Opaque description of one diagonal pattern: shape, offset table, and the
 * device-resident run table the tiled kernels walk.  Replaces the contents of
 * dev_block_descriptor (src/cuv/matrix_ops/densedense_to_sparse.hpp:69-105,
 * built in densedense_to_sparse.cu:123-171) -- O(num_dia) instead of one
 * entry per 16x16 block -- and the device copy of dia_matrix::m_offsets
 * (src/cuv/basics/dia_matrix.hpp:75). */
typedef struct cuvdia_desc cuvdia_desc;

/* Builds a descriptor from a HOST offset table (table order is preserved:
 * vals slot d belongs to offsets_host[d]).  Requires nd >= 1, h, w >= 1,
 * row_fact >= 1 and stride >= h or stride >= w (dia_matrix.hpp:106,131).
 * Allocates a few KB of device memory. */
int cuvdia_desc_create(cuvdia_desc **out, const int *offsets_host, int nd,
                       int h, int w, int stride, int row_fact);

/* Frees the descriptor and its device table.  NULL is accepted. */
int cuvdia_desc_destroy(cuvdia_desc *desc);

/* Host-side facts about a descriptor (any pointer may be NULL):
 * number of run chunks the products walk for the normal and the transposed
 * traversal (cuvdia_plan_chunks_max with max_len 13), and the number of
 * valid (non-padding) elements. */
int cuvdia_desc_info(const cuvdia_desc *desc, int *chunks_n, int *chunks_t,
                     long long *nnz);

/* Pure host function (no GPU needed): decomposes an offset table into the
 * run chunks the tiled kernels walk.  Shifts are the offsets themselves
 * (transposed == 0) or their negation (transposed != 0), sorted ascending;
 * a run is a maximal sequence of consecutive shifts and is cut into
 * near-equal chunks of at most max_len, 1 <= max_len <= 13.  The products
 * walk the tables of max_len 13 (one staged block of 76 dense rows serves 64
 * output rows and 13 shifts), the dense x dense^T projection the table of
 * max_len 8, transposed == 0.  Chunk c covers shifts s0[c] .. s0[c]+len[c]-1
 * and slot[max_len*c + j] is the table position of the j-th one (-1 for
 * j >= len[c]).  Returns the number of chunks (also when it exceeds cap; then
 * nothing is written), or a negative error. */
int cuvdia_plan_chunks_max(const int *offsets_host, int nd, int transposed, int max_len,
                           int *s0, int *len, int *slot, int cap);

/* cuvdia_plan_chunks_max with max_len 8. */
int cuvdia_plan_chunks(const int *offsets_host, int nd, int transposed,
                       int *s0, int *len, int *slot, int cap);

/* Pure host function: the work units the tiled dense x dense^T projection
 * walks.  A unit is one chunk of the normal (transposed == 0) chunk table, or
 * two chunks adjacent in that table whose first shifts differ by a positive
 * multiple of 4 of at most 4096 rows (two rows of a 2-d window): up to 256
 * rows apart a wave serves both from one staged band of the second operand and
 * one copy of the first operand's rows; further apart the second chunk works
 * on the rows that far above the first's, so that both read the same rows of
 * the second operand.  c1[u] is the unit's chunk
 * index, c2[u] its second chunk or -1.  Returns the number of units (also when
 * it exceeds cap; then nothing is written), or a negative error.  The role of
 * the block list built in src/cuv/matrix_ops/densedense_to_sparse.cu:123-171. */
int cuvdia_plan_units(const int *offsets_host, int nd, int *c1, int *c2, int cap);

/* Pure host function: does the automatic choice of cuvdia_dd2dia_f32 run the
 * kernel tiled in the window's plane for an h x w matrix with this table
 * (row_fact 1) and `batch` packed dense columns?  Returns the number of
 * workgroups of that launch (tiles of 4 x 64 positions x blocks of 8 window
 * rows -- of 7 where a window row has 9 to 13 diagonals, or of 5 where that
 * leaves fewer rows of the last block empty and the staging buffers of three
 * workgroups fit a CU's LDS -- x channel groups), or 0 when the chunk-by-chunk kernel serves: the table is no
 * window table (see cuvdia_plan_walk) of chunks of 2 to 13 diagonals, the
 * period, a channel distance or a row count is no multiple of 4, the period
 * is below 64, or the launch has too few workgroups to fill the chip.  For
 * chunks of up to 8 diagonals: 768 for windows of 49 slots or more -- or 384
 * at a batch of at least 512, or 192 at a batch of at least 32: a workgroup
 * then works two or four ranges of the batch side by side --, 1024 from 25
 * slots, 1536 and a batch of at least 128 below.  For chunks of 9 to 13, on
 * periods of at least 192: 4096; or 1024 (512 on periods of at least 256)
 * when the blocks of window rows are at least nine tenths full (13 and 14
 * rows; 9, 10 and 15 in blocks of 5); or 1024 when window rows x channel
 * groups are at least 22.
 * Negative: an error.
 * cuvdia_set_path(CUVDIA_PATH_WINDOW) waives the conditions on the period's
 * size, the workgroups and the batch.  No counterpart in the reference. */
long long cuvdia_plan_window_launch(const int *offsets_host, int nd, int stride, int h, int w, int batch);

/* Pure host function: is the offset table a *window table* -- k window rows of
 * lck consecutive offsets, `period` rows apart, repeated for every one of
 * ngroups groups (channel shifts); the pattern filter_factory builds
 * (src/cuv/basics/filter_factory.hpp:43-91) -- and does the walking product
 * kernel serve it?  transposed selects the table of the transposed product.
 * Writes period, k, ngroups and lck (each pointer may be NULL) when the answer
 * is not 0.  Returns 0: no window table; 1: a window table that the products
 * walk tile by tile (with their row tiles numbered period-major on launches of
 * many rounds); 2: a window table with a walking kernel (centred 3x3, 5x5 or
 * 7x7 window, period a multiple of 64); negative: an error.  The answer is
 * about the TABLE only.  Whether a given product runs the walking kernel also
 * depends on its shape -- cuvdia_plan_walk_launch answers that.  No
 * counterpart in the reference. */
int cuvdia_plan_walk(const int *offsets_host, int nd, int stride, int transposed,
                     int *period, int *k, int *ngroups, int *lck);

/* Pure host function: does the automatic choice of cuvdia_spmm_f32 -- and of
 * cuvdia_spmm_bias_act_f32 and cuvdia_spmm_layer_f32: the bias, the sigmoid
 * and the sample are applied where the walking kernel's tiles leave -- run
 * the walking kernel for the product of an h x w
 * matrix with this table (row_fact 1) and `batch` packed dense columns?
 * Returns the number of workgroups of that launch, or 0 when another kernel
 * serves: the table is no window table with a walking kernel (see
 * cuvdia_plan_walk), the output row count is no multiple of 64 or the input
 * row count no multiple of 4, batch < 24, or the launch would have fewer than
 * 384 workgroups (a product of few tiles is served tile by tile).  Negative:
 * an error.  cuvdia_set_path(CUVDIA_PATH_WALK) waives the last condition
 * only.  No counterpart in the reference. */
long long cuvdia_plan_walk_launch(const int *offsets_host, int nd, int stride, int h, int w,
                                  int transposed, int batch);

/* dst = beta*dst + alpha*op(A)*B for a batch of dense columns.
 * Replaces prod<float,dev_memory_space,column_major>(dst, dia A, B, transA,
 * 'n', factAB, factC) (src/cuv/matrix_ops/spmv.cu:221-247), the spmv it
 * forwards to (spmv.cu:89-101,130-139) and the generated kernel dispatcher
 * (src/cuv/matrix_ops/make_spmv_header.pl:94-127, kernels in
 * src/cuv/matrix_ops/spmv_kernel.cuh:55-300).
 *   transA == 'n': A is h x w, B is w x batch (ldb >= w), dst h x batch (ldd >= h)
 *   transA == 't': B is h x batch (ldb >= h), dst is w x batch (ldd >= w)
 * beta == 0 follows the reference HOST rule (spmv.cu:152-156): dst is
 * overwritten and never read, so it may hold NaN.  batch == 0 is a no-op.
 * B and dst must not overlap.
 * Non-finite values in B: every kernel family multiplies exactly the stored
 * elements, as the reference's host loop does (spmv.cu:183-197): an Inf or
 * NaN in a row of B reaches the result rows that reference that row and no
 * other (chunks shorter than the table's longest run only the diagonals
 * they have). */
int cuvdia_spmm_f32(const cuvdia_desc *desc, const float *A_vals_device,
                    const float *B_device, long long ldb,
                    float *dst_device, long long ldd, int batch,
                    char transA, float alpha, float beta, void *stream);

/* The same product with the two element-wise passes an RBM/MLP layer runs on
 * its result fused into the store:
 *   dst = act(beta*dst + alpha*op(A)*B + bias[row])
 * i.e. prod (above), then matrix_plus_col(dst, bias)
 * (src/cuv/matrix_ops/matrix_ops.hpp:307), then apply_scalar_functor(dst, SIGM)
 * (src/cuv/tensor_ops/functors.hpp:122) as in examples/rbm/base.py:48-54,127-136.
 * bias: device array with one float per output row, or NULL for none;
 * act: CUVDIA_ACT_NONE or CUVDIA_ACT_SIGMOID.  With bias == NULL and
 * CUVDIA_ACT_NONE this is cuvdia_spmm_f32.  batch == 0 is a no-op. */
int cuvdia_spmm_bias_act_f32(const cuvdia_desc *desc, const float *A_vals_device,
                             const float *B_device, long long ldb,
                             float *dst_device, long long ldd, int batch,
                             char transA, float alpha, float beta,
                             const float *bias_device, int act, void *stream);

/* The layer update with a Bernoulli sample of the result:
 *   p = 1/(1+exp(-(beta*dst + alpha*op(A)*B + bias[row]))),
 *   dst = p > u(row, col) ? 1 : 0                    (act == CUVDIA_ACT_SIGMOID_SAMPLE)
 * -- prod, matrix_plus_col, SIGM and rnd_binarize (src/cuv/random/random.cu:86-91,
 * 139-142: f > uniform) of examples/rbm/base.py:48-54,94-99,127-136 in one
 * launch.  The reference draws u from cuRAND's per-thread XORWOW states (a
 * closed third-party generator whose stream depends on the launch shape);
 * here u(row, col) = (w >> 8) * 2^-24 with w = word (col & 3) of
 * Philox4x32-10 (Salmon et al., SC'11) at counter (row, col >> 2, 0, 0) and
 * key (seed & 0xffffffff, seed >> 32): a function of the seed and the
 * element's position in dst only, so results do not depend on the kernel
 * family or the tiling.  row, col index dst (0-based).  With CUVDIA_ACT_NONE or
 * CUVDIA_ACT_SIGMOID this is cuvdia_spmm_bias_act_f32 and the seed is unused.
 * No counterpart with this signature exists in the reference. */
int cuvdia_spmm_layer_f32(const cuvdia_desc *desc, const float *A_vals_device,
                          const float *B_device, long long ldb,
                          float *dst_device, long long ldd, int batch,
                          char transA, float alpha, float beta,
                          const float *bias_device, int act,
                          unsigned long long seed, void *stream);

/* W[i] = -learnrate*dW[i] + (1 - learnrate*decay)*W[i] for i < n: replaces
 * learn_step_weight_decay<float,dev_memory_space>
 * (src/cuv/tensor_ops/rprop.cu:148-156,324-346, declared in
 * src/cuv/tensor_ops/rprop.hpp:127-128; the reference ignores sparsedecay,
 * rprop.cu:153-154).  For a DIA weight matrix W and dW are the value vectors
 * (num_dia*stride floats, padding included, as the reference's call on
 * dia.vec() does).  W and dW must not overlap.  n == 0 is a no-op.
 * When dW is itself a projected product, cuvdia_dd2dia_f32 with
 * alpha = -learnrate*scale and beta = 1 - learnrate*decay applies the same
 * update without materialising dW. */
int cuvdia_learn_step_weight_decay_f32(float *W_device, const float *dW_device, long long n,
                                       float learnrate, float decay, void *stream);

/* m = momentum_weight*momentum[i] - learnrate*(dW[i] + decay*W[i]);
 * W[i] += m; momentum[i] = m, for i < n: replaces
 * learn_step_weight_decay_momentum<float,dev_memory_space>
 * (src/cuv/tensor_ops/rprop.cu:158-170,348-353,369-376, declared in
 * src/cuv/tensor_ops/rprop.hpp:142-143; sparsedecay is ignored there,
 * rprop.cu:166-167).  The reference's host loop (rprop.cu:356-367) has the
 * decay term with the opposite sign; this entry follows the device kernel it
 * replaces, which is the one that shrinks the weights.  The three arrays must
 * not overlap.  n == 0 is a no-op. */
int cuvdia_learn_step_weight_decay_momentum_f32(float *W_device, float *momentum_device,
                                                const float *dW_device, long long n,
                                                float learnrate, float momentum_weight,
                                                float decay, void *stream);

/* C = beta*C + alpha*proj(A*B') restricted to the stored diagonals of C:
 *   C_d[i] = beta*C_d[i] + alpha * sum_c A[i,c] * B[offsets[d] + i/row_fact, c]
 * for every valid slot.  Replaces densedense_to_dia<float,column_major>
 * (dev) (src/cuv/matrix_ops/densedense_to_sparse.cu:253-308) and its kernel
 * dense2dia_mm (densedense_to_sparse.cu:51-120), with the documented
 * contract of src/cuv/matrix_ops/densedense_to_sparse.hpp:107-121.
 * A is h x batch (lda >= h), B is w x batch (ldb >= w).  beta == 0 never
 * reads C.  batch == 0 scales C by beta (zero-fills valid slots if beta == 0).
 * A batch whose operands are larger than 2 GiB is worked in several launches
 * on `stream`, slab of columns after slab, each adding to C.
 * Summation order per slot: see kernels.hip; the kernel for large window
 * tables (cuvdia_last_path() == CUVDIA_PATH_WINDOW) adds the batch columns in
 * ascending order into one sum (on launches of few tiles of a window with
 * rows of at most 8 diagonals: into two or four sums over consecutive ranges
 * of the batch), the chunk-by-chunk kernel into
 * four or eight interleaved partial sums: their results differ by rounding,
 * both within 1e-5 of the sum of |terms| of the reference's host result. */
int cuvdia_dd2dia_f32(const cuvdia_desc *desc, float *C_vals_device,
                      const float *A_device, long long lda,
                      const float *B_device, long long ldb, int batch,
                      float alpha, float beta, void *stream);

/* dst[d] = mean of stored diagonal d over its valid (non-padding) slots, for
 * every table position d; dst is a device array of num_dia floats.  Replaces
 * avg_diagonals<float,dev_memory_space> (src/cuv/matrix_ops/diagonals.cu:14-22,
 * declared in src/cuv/matrix_ops/diagonals.hpp:12) with the semantics of the
 * host version (diagonals.cu:24-51: the mean over the N_d = min(h - max(0,-k),
 * w - max(0,k)) valid slots, padding never read; the reference's device
 * version averages over the padded stride instead, so ITS NUMBERS DIFFER
 * from this entry's for every off-centre diagonal: sum/stride there,
 * sum/N_d here).  row_fact must be 1
 * (diagonals.cu:28), else CUVDIA_EUNSUPPORTED; a diagonal without valid slots
 * yields 0. */
int cuvdia_avg_diagonals_f32(const cuvdia_desc *desc, const float *A_vals_device,
                             float *dst_device, void *stream);

/* The same two operations taking the offset table from HOST memory on every
 * call, for callers that hold only a dia_matrix (the reference signatures
 * carry no descriptor for prod).  A descriptor is created on first sight of
 * an (offsets, h, w, stride, row_fact) combination and kept in a small
 * process-wide cache (device allocation on a miss only). */
int cuvdia_spmm_offsets_f32(const float *A_vals_device, const int *offsets_host,
                            int nd, int stride, int h, int w, int row_fact,
                            const float *B_device, long long ldb,
                            float *dst_device, long long ldd, int batch,
                            char transA, float alpha, float beta, void *stream);

int cuvdia_dd2dia_offsets_f32(float *C_vals_device, const int *offsets_host,
                              int nd, int stride, int h, int w, int row_fact,
                              const float *A_device, long long lda,
                              const float *B_device, long long ldb, int batch,
                              float alpha, float beta, void *stream);

/* cuvdia_spmm_offsets_f32 for callers that cannot allocate device memory:
 * code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference.  Same arguments, same
 * argument rules, and the generic or tile-by-tile kernels chosen as there:
 * bit-identical results wherever cuvdia_spmm_offsets_f32 does not take its
 * walking kernel (large products of window tables; CUVDIA_PATH_TILED_NOWALK
 * keeps it from doing so), within rounding of them where it does.  But the
 * device copy of the offset table and of the chunk table the kernels walk -- which a
 * descriptor keeps in memory it allocates -- lives in a static device array
 * of 20480 bytes inside the library (one copy per GPU, held until the process
 * ends), so the call allocates and frees no DEVICE memory -- no hipMalloc, no
 * hipFree, no allocating library call -- and touches neither the descriptor
 * cache nor its lock.  (It does plan the chunk table on the host, in a small
 * std::vector on the host heap.)  The first call on a GPU also resolves the
 * array's address there (hipGetSymbolAddress, which may load the library's
 * code object): make that first call outside stream capture; every later
 * call on that GPU may be captured.  Every
 * call rewrites the part of the array it uses with one small fill kernel per
 * 3584 bytes of table, enqueued on `stream` ahead of the product (the bytes
 * travel as kernel arguments, so the host table may be reused on return).
 * Capacity: nd <= 1024, else CUVDIA_ETOOLARGE (nothing is enqueued); a table
 * of more than 256 chunks is served by the generic kernels, as everywhere.
 * All calls on one GPU share that GPU's array: calls ordered on one stream
 * are safe, calls that may overlap (different streams or host threads without
 * ordering between them) race on it. */
int cuvdia_spmm_offsets_noalloc_f32(const float *A_vals_device, const int *offsets_host,
                                    int nd, int stride, int h, int w, int row_fact,
                                    const float *B_device, long long ldb,
                                    float *dst_device, long long ldd, int batch,
                                    char transA, float alpha, float beta, void *stream);

/* Drops every descriptor held by the *_offsets_* cache. */
int cuvdia_cache_clear(void);

/* Forces a kernel family for subsequent calls (process-wide; tests use it to
 * run both families on the same inputs).  CUVDIA_PATH_TILED on a request the
 * tiled kernels cannot serve (row_fact > 1) returns CUVDIA_EUNSUPPORTED from
 * the compute call.  CUVDIA_PATH_WALK, CUVDIA_PATH_WINDOW and
 * CUVDIA_PATH_TILED_NOWALK choose inside the tiled family: a kernel for
 * window tables whatever the size of the operands, or none of them.
 * CUVDIA_PATH_WALK: the walking product (CUVDIA_EUNSUPPORTED for a table
 * that is no window table with a walking kernel; densedense_to_dia treats it
 * as CUVDIA_PATH_TILED_NOWALK).  CUVDIA_PATH_WINDOW: the kernels tiled in the
 * window's plane, which serve densedense_to_dia (CUVDIA_EUNSUPPORTED when
 * they do not serve the request: no window table of chunks of 2 to 13
 * diagonals, a period, channel distances or row counts that are no multiples
 * of 4); the products treat it as CUVDIA_PATH_TILED_NOWALK. */
int cuvdia_set_path(int path);

/* Which family the most recent compute call on this thread launched
 * (CUVDIA_PATH_GENERIC, CUVDIA_PATH_TILED, CUVDIA_PATH_WALK for a product
 * served by the walking kernel, CUVDIA_PATH_WINDOW for a projection served
 * by the kernel tiled in the window's plane; 0 before any call). */
int cuvdia_last_path(void);

/* Name of the kernel the most recent compute call on this thread launched
 * (the last one, where a call launches several), written as a profiler
 * prints it, e.g. "spmm_tiled_kernel<7, 8, 1, false>"; "" before any call.
 * The string belongs to the library and is overwritten by the next call.
 * No counterpart in the reference. */
const char *cuvdia_last_kernel(void);

/* Static string for an error code. */
const char *cuvdia_strerror(int code);

/* Text of the last HIP failure seen by this thread ("" if none). */
const char *cuvdia_last_hip_error(void);

/* ABI revision of this header. */
int cuvdia_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* CUVDIA_H */
