// Launch interface between the C ABI (api.cpp) and the gfx950 kernels
// (kernels.hip).  Everything here is host-callable; shapes have been validated
// by the caller.
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstddef>

#include "plan.hpp"

namespace cuvdia {

// Device form of a window table (plan_walk) for one traversal; tab_dev == nullptr: not a window table.
struct WalkView {
    const int *tab_dev;          // group_rows[ngroups], then aoff4[ngroups * k]
    int ngroups, period, s0, k, lck, astep4;
    bool rows4;                  // every group_rows[g] is a multiple of 4
};

struct DiaView {
    int h, w, nd, stride, rf;
    const int *offsets_dev;      // nd ints, table order
    const Chunk *chunks_n_dev;   // the products' tables (chunks of up to SP_CHUNK_MAX): shifts = offsets
    int n_chunks_n;
    const Chunk *chunks_t_dev;   // shifts = -offsets
    int n_chunks_t;
    int max_len_n, max_len_t;    // longest chunk of each table
    int min_len_n, min_len_t;    // shortest chunk of each table
    int s_min_n, s_max_n;        // smallest / largest chunk shift of each table
    int s_min_t, s_max_t;
    int slot_step_n, slot_step_t; // common_slot_step of each table (0: none)
    WalkView walk_n, walk_t;     // window-table form of the two products' tables
    const Chunk *chunks_p_dev;   // the projection's table (chunks of up to CHUNK_MAX): shifts = offsets
    int n_chunks_p;
    int max_len_p;
    const Unit *units_dev;       // units of the normal table (dense x dense^T projection)
    int n_units;
    int pair_delta_max;          // largest distance between the first shifts of a pair (0: no pairs)
    const Unit *single_units_dev;   // one unit per chunk of the normal table, in table order
};

// What the SpMM kernels do to a result element before storing it:
// v = beta*dst + alpha*sum; v += bias[row] (bias != nullptr); v = 1/(1+exp(-v))
// (act >= 1); v = v > u(row, col) ? 1 : 0 (act == 2), u being the uniform
// variate in [0, 1) that sp_uniform() derives from (seed, row, col) with
// Philox4x32-10.  The default, {nullptr, 0, 0, 0}, stores the plain product.
struct SpEpilogue {
    const float *bias;   // one value per output row, on the device, or nullptr
    int act;             // 0: none, 1: logistic sigmoid, 2: sigmoid, then a Bernoulli sample of it
    unsigned seed_lo, seed_hi;
};

// dst = beta*dst + alpha*op(A)*B.  One thread per output row, a few batch
// columns per thread; honours row_fact.
hipError_t launch_spmm_generic(const DiaView &A, const float *vals, const float *B, long long ldb,
                               float *dst, long long ldd, int batch, bool trans,
                               float alpha, float beta, SpEpilogue ep, hipStream_t stream);

// Same contract, row_fact == 1 only: 64 output rows x 64 batch columns per
// workgroup, dense tile staged through LDS once per run chunk, lanes own
// batch columns and keep a sliding register window along the rows, diagonal
// values are broadcast across each 16-lane row by DPP.  Window tables on
// products of many tiles go to the walking kernel, which stages a block of
// dense rows once for all the window rows that read it.  `walk`: 0 -- that
// choice is made by size; 1 -- the walking kernel or hipErrorNotSupported;
// -1 -- never the walking kernel.  *walked (if not null) tells which ran.
// Output rows per tile of the walking kernel's instantiation for a window of k rows of lck diagonals whose first
// shift is s0; 0 when there is none.
// Records the name of the kernel a launcher is about to launch, written the way a profiler prints it
// ("spmm_tiled_kernel<7, 8, 1, false>"), for cuvdia_last_kernel(); per host thread.
void note_kernel(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
int spmm_walk_tile_rows(int lck, int k, int s0);
// Tiles per segment of the walking launch for such a window on n_out x n_in rows and col_tiles tiles of 64 batch
// columns, and the launch's workgroups; 0 when the walking kernel does not run there (no instantiation, row
// counts its tiles do not divide, or -- unless forced -- too few workgroups to fill the chip).
int spmm_walk_plan(int lck, int k, int s0, int period, long long n_out, long long n_in, long long col_tiles,
                   bool forced, long long *workgroups);
hipError_t launch_spmm_tiled(const DiaView &A, const float *vals, const float *B, long long ldb,
                             float *dst, long long ldd, int batch, bool trans,
                             float alpha, float beta, SpEpilogue ep, hipStream_t stream,
                             int walk = 0, bool *walked = nullptr);

// m = mw*M[i] - lr*(dW[i] + l2*W[i]); W[i] += m; M[i] = m, i < n.
hipError_t launch_momentum(float *W, float *M, const float *dW, long long n, float lr, float mw, float l2,
                           hipStream_t stream);

// W[i] = alpha*dW[i] + beta*W[i], i < n.
hipError_t launch_axpby(float *W, const float *dW, long long n, float alpha, float beta, hipStream_t stream);

// Whether the tiled SpMM can serve these operands (row_fact 1, operand extents
// within its 32-bit buffer addressing).
bool spmm_tiled_ok(const DiaView &A, long long ldb, long long ldd, bool trans);

// C_d[i] = beta*C_d[i] + alpha*sum_c A[i,c]*B[k_d + i/rf, c] on valid slots.
// One thread per slot, serial over the batch; honours row_fact.
hipError_t launch_dd2dia_generic(const DiaView &C, float *vals, const float *A, long long lda,
                                 const float *B, long long ldb, int batch,
                                 float alpha, float beta, hipStream_t stream);

// Whether the tiled dd2dia can serve these operands (row_fact 1, operand
// extents within its 32-bit buffer addressing).
bool dd2dia_tiled_ok(const DiaView &C, long long lda, long long ldb, int batch);
// The largest number of batch columns (a multiple of 32) whose rows of both operands lie within the tiled
// kernel's 32-bit byte offsets, 0 if not even DD2DIA_SLAB_MIN do.
constexpr int DD2DIA_SLAB_MIN = 32;
int dd2dia_slab_columns(const DiaView &C, long long lda, long long ldb);

// Same contract, row_fact == 1 only: a workgroup owns 256 rows of one run
// chunk; each lane keeps 4 rows x (longest chunk) diagonals of partial sums,
// the four waves split the batch and are summed through LDS in wave order.
// Window tables whose tiles fill the chip go to the window-table projection (a tile of 4 x 64 positions of the
// window's plane per workgroup, both operands staged once for all the slots of up to 8 window rows).
// `window`: 0 -- that choice is made by size; 1 -- that kernel or hipErrorNotSupported; -1 -- never.
// *windowed (if not null) tells which ran.
hipError_t launch_dd2dia_tiled(const DiaView &C, float *vals, const float *A, long long lda,
                               const float *B, long long ldb, int batch,
                               float alpha, float beta, hipStream_t stream, int window = 0, bool *windowed = nullptr);
// Workgroups of the window-table projection for these operands (0: it does not apply).
long long dd2dia_window_workgroups(const DiaView &C, int batch, int *txn = nullptr, int *tyn = nullptr, int *ndb = nullptr);
// Whether the automatic choice takes that kernel for a launch of so many workgroups.
bool dd2dia_window_by_size(const DiaView &C, int batch, long long workgroups);
// Batch ranges per workgroup (1, 2 or 4) of such a launch.
int dd2dia_window_subs(const DiaView &C, long long workgroups);

// The allocation-free entry point keeps its device tables in a static device
// array instead of a descriptor's allocation: the offset table at byte 0 (up
// to NOALLOC_MAX_DIAGONALS ints), one chunk table at NOALLOC_CHUNKS_AT (up to
// NOALLOC_MAX_CHUNKS entries of 64 bytes).
constexpr int NOALLOC_MAX_DIAGONALS = 1024;
constexpr int NOALLOC_MAX_CHUNKS = 256;
constexpr size_t NOALLOC_CHUNKS_AT = (size_t)NOALLOC_MAX_DIAGONALS * sizeof(int);
constexpr size_t NOALLOC_SCRATCH_BYTES = NOALLOC_CHUNKS_AT + (size_t)NOALLOC_MAX_CHUNKS * sizeof(Chunk);
constexpr size_t NOALLOC_PIECE_BYTES = 3584;     // table bytes one fill launch carries in its kernel arguments
// Address of that array on the current device (looked up once per device).
hipError_t noalloc_scratch(unsigned char **out);
// Enqueues the copy of `bytes` (a multiple of 4) host bytes to dst_dev, a place
// inside the array, on `stream`: the bytes travel as kernel arguments, so no
// staging buffer is allocated and src_host may be reused on return.
hipError_t noalloc_upload(unsigned char *dst_dev, const void *src_host, size_t bytes, hipStream_t stream);

// dst[d] = mean of diagonal d over its valid slots (row_fact == 1), dst on the device.
hipError_t launch_avg_diagonals(const DiaView &A, const float *vals, float *dst, hipStream_t stream);

}  // namespace cuvdia
