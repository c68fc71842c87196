// gfx950 (MI355X, CDNA4) kernels for products with diagonal-sparse matrices.
//
// Two families per operation:
//   generic -- one thread per output element, guards everywhere, any row_fact;
//              the shape of the reference's own kernels
//              (src/cuv/matrix_ops/spmv_kernel.cuh:114-172) and the correctness
//              anchor on the GPU;
//   tiled   -- row_fact == 1, wave64 register-blocked kernels described at
//              each kernel below.
//
// Accumulation order (fp32, fused multiply-add, per output element):
//   spmm    acc = 0; for each run chunk in ascending shift order, for each
//           diagonal of the chunk in ascending shift order:
//           acc = fma(a, x, acc); then dst = beta*dst + alpha*acc
//           (dst = alpha*acc when beta == 0, dst never read).
//           The generic kernel walks the offset table in table order instead.
//   dd2dia  four partial sums, wave q of the workgroup owning batch columns
//           {4*g + i : g = q (mod 4), i < 4} in ascending order, each
//           acc = fma(a, b, acc); total = ((p0 + p1) + p2) + p3;
//           C = beta*C + alpha*total.  The generic kernel sums the batch
//           serially in ascending column order.
#include <hip/hip_runtime.h>

#include "kernels.hpp"

namespace cuvdia {
namespace {

// Loads through this address space are issued on the scalar unit when the
// address is wave-uniform: diagonal values and the chunk table reach the
// FMAs as SGPR operands and cost no vector-memory or LDS bandwidth.
typedef const float __attribute__((address_space(4))) *sc_float_ptr;
typedef const Chunk __attribute__((address_space(4))) *sc_chunk_ptr;

__device__ __forceinline__ sc_float_ptr scalar_ptr(const float *p) { return (sc_float_ptr)p; }
__device__ __forceinline__ sc_chunk_ptr scalar_ptr(const Chunk *p) { return (sc_chunk_ptr)p; }

// Hardware hands consecutive workgroup ids to the 8 XCDs round-robin, and each
// XCD has its own L2.  Remap so that every XCD works on one contiguous span of
// tiles: neighbouring row tiles share dense-operand rows (the halo and the
// bands +-px apart), which then hit in that XCD's L2.
__device__ __forceinline__ int xcd_tile(int bid, int nblk)
{
    constexpr int XCDS = 8;
    const int q = nblk / XCDS, r = nblk % XCDS;
    const int xcd = bid % XCDS, slot = bid / XCDS;
    return xcd * q + (xcd < r ? xcd : r) + slot;
}

// Orders this wave's LDS writes before its later LDS reads (and the reverse)
// for data exchanged between lanes of ONE wave.  The LDS unit executes a
// wave's instructions in order, so only the compiler needs restraining.
__device__ __forceinline__ void wave_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ------------------------------------------------------------------ generic --

template <int CB>
__global__ __launch_bounds__(256) void spmm_generic_kernel(
    const int *__restrict__ offsets, int nd, const float *__restrict__ vals, int stride,
    int h, int w, int rf, const float *__restrict__ X, long long ldx,
    float *__restrict__ Y, long long ldy, int n_out, int batch, int trans,
    float alpha, float beta)
{
    const long long o = (long long)blockIdx.x * 256 + threadIdx.x;
    const int c0 = blockIdx.y * CB;
    if (o >= n_out) return;
    float acc[CB];
#pragma unroll
    for (int c = 0; c < CB; ++c) acc[c] = 0.f;

    for (int d = 0; d < nd; ++d) {
        const long long k = offsets[d];
        const float *vd = vals + (long long)d * stride;
        if (!trans) {
            // src/cuv/matrix_ops/spmv.cu:183-197
            const long long i_start = rf * (k < 0 ? -k : 0);
            const long long j_start = k > 0 ? k : 0;
            const long long N = min((long long)h - i_start, rf * ((long long)w - j_start));
            const long long n = o - i_start;
            if (n >= 0 && n < N) {
                const float a = vd[o];
                const long long col = j_start + n / rf;
#pragma unroll
                for (int c = 0; c < CB; ++c)
                    if (c0 + c < batch)
                        acc[c] = __builtin_fmaf(a, X[(long long)(c0 + c) * ldx + col], acc[c]);
            }
        } else {
            // src/cuv/matrix_ops/spmv.cu:161-177
            const long long i_start = k > 0 ? k : 0;
            const long long j_start = rf * (k < 0 ? -k : 0);
            const long long N = min(((long long)h - j_start) / rf, (long long)w - i_start);
            const long long n = o - i_start;
            if (n >= 0 && n < N) {
                for (int q = 0; q < rf; ++q) {
                    const long long r = j_start + n * rf + q;
                    const float a = vd[r];
#pragma unroll
                    for (int c = 0; c < CB; ++c)
                        if (c0 + c < batch)
                            acc[c] = __builtin_fmaf(a, X[(long long)(c0 + c) * ldx + r], acc[c]);
                }
            }
        }
    }
#pragma unroll
    for (int c = 0; c < CB; ++c) {
        if (c0 + c < batch) {
            float *y = Y + (long long)(c0 + c) * ldy + o;
            *y = (beta == 0.f) ? alpha * acc[c] : beta * (*y) + alpha * acc[c];
        }
    }
}

__global__ __launch_bounds__(256) void dd2dia_generic_kernel(
    const int *__restrict__ offsets, float *__restrict__ C, int stride, int h, int w, int rf,
    const float *__restrict__ A, long long lda, const float *__restrict__ B, long long ldb,
    int batch, float alpha, float beta)
{
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;   // slot within the diagonal == row
    const int d = blockIdx.y;
    // src/cuv/matrix_ops/densedense_to_sparse.cu:221-227
    const long long k = offsets[d];
    const long long row_start = rf * (k < 0 ? -k : 0);
    const long long col_start = k > 0 ? k : 0;
    const long long N = min((long long)h - row_start, rf * ((long long)w - col_start));
    const long long n = i - row_start;
    if (n < 0 || n >= N) return;
    const float *a = A + i;
    const float *b = B + col_start + n / rf;
    float s = 0.f;
    for (int c = 0; c < batch; ++c)
        s = __builtin_fmaf(a[(long long)c * lda], b[(long long)c * ldb], s);
    float *dst = C + (long long)d * stride + i;
    *dst = (beta == 0.f) ? alpha * s : beta * (*dst) + alpha * s;
}

// -------------------------------------------------------------- tiled spmm --
//
// Workgroup = 64 output rows x 64 batch columns, WAVES waves of T = 64/WAVES
// rows each.  Lane l of every wave owns batch column col0 + l and T running
// sums.  Per run chunk (<= 8 consecutive shifts starting at s0):
//   1. the dense rows [row0 + s0, row0 + s0 + 72) of the 64 columns are
//      loaded with lanes along rows (coalesced 256-byte segments) and written
//      to LDS column by column, pitch 76 floats;
//   2. each lane reads its column's window of T + len - 1 values with 16-byte
//      LDS reads (pitch/4 is odd, so the 64 lanes spread over all banks);
//   3. for each diagonal j and row t: acc[t] = fma(A_j[row], win[t + j], acc[t])
//      where A_j[row] is wave-uniform and arrives as an SGPR operand.
// The next chunk's global loads are issued before the FMAs of the current one
// and written to the other LDS buffer afterwards (one barrier per chunk).
// The epilogue transposes the sums through LDS so the store to dst is again
// lanes-along-rows.

constexpr int SP_ROWS = 64;        // output rows per workgroup
constexpr int SP_COLS = 64;        // batch columns per workgroup (one per lane)
constexpr int SP_STAGED = 72;      // rows staged per chunk: 64 + CHUNK_MAX
constexpr int SP_PITCH = 76;       // floats between staged columns
constexpr int SP_OPITCH = 68;      // floats between columns in the epilogue

template <int T, int LC, bool GUARD>
__device__ __forceinline__ void spmm_chunk(float (&acc)[T], const float *win_lds,
                                           sc_float_ptr vals, sc_chunk_ptr ck, int s0,
                                           long long stride, long long arow, int ashift,
                                           int n_out, int n_in)
{
    constexpr int WIN = T + LC - 1;
    constexpr int WQ = (WIN + 3) / 4;
    float win[WQ * 4];
    const float4 *p4 = reinterpret_cast<const float4 *>(win_lds);
#pragma unroll
    for (int q = 0; q < WQ; ++q) {
        const float4 v = p4[q];
        win[4 * q + 0] = v.x; win[4 * q + 1] = v.y; win[4 * q + 2] = v.z; win[4 * q + 3] = v.w;
    }
#pragma unroll
    for (int j = 0; j < LC; ++j) {
        const long long abase = (long long)ck->slot[j] * stride + arow + (ashift ? s0 + j : 0);
#pragma unroll
        for (int t = 0; t < T; ++t) {
            float a;
            if (!GUARD) {
                a = vals[abase + t];
            } else {
                const long long o = arow + t;
                const long long in = o + s0 + j;
                const bool ok = (o < n_out) & (in >= 0) & (in < n_in);
                a = vals[ok ? abase + t : 0];
                a = ok ? a : 0.f;
            }
            acc[t] = __builtin_fmaf(a, win[t + j], acc[t]);
        }
    }
}

template <int T, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void spmm_tiled_kernel(
    const Chunk *__restrict__ chunks, int nchunks, const float *__restrict__ vals, int stride,
    int ashift, const float *__restrict__ X, long long ldx, float *__restrict__ Y, long long ldy,
    int n_out, int n_in, int batch, float alpha, float beta, int col_tiles)
{
    static_assert(T * WAVES == SP_ROWS, "a workgroup covers 64 rows");
    constexpr int CPW = SP_COLS / WAVES;        // columns each wave stages
    constexpr int HALO = (CPW + 7) / 8;         // halo loads per wave (8 rows x 8 columns each)
    __shared__ __attribute__((aligned(16))) float lds[2][SP_COLS * SP_PITCH];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tile = xcd_tile(blockIdx.x, gridDim.x);
    const int rowtile = tile / col_tiles;
    const int row0 = rowtile * SP_ROWS;
    const int col0 = (tile - rowtile * col_tiles) * SP_COLS;
    const sc_chunk_ptr cks = scalar_ptr(chunks);
    const sc_float_ptr svals = scalar_ptr(vals);

    float acc[T];
#pragma unroll
    for (int t = 0; t < T; ++t) acc[t] = 0.f;
    float pre[CPW + HALO];

    const int hcol = lane >> 3, hrow = SP_ROWS + (lane & 7);

    auto issue = [&](int c) {
        const long long base = (long long)row0 + cks[c].s0;
        const bool interior = (base >= 0) & (base + SP_STAGED <= n_in) & (col0 + SP_COLS <= batch);
        if (interior) {
#pragma unroll
            for (int q = 0; q < CPW; ++q)
                pre[q] = X[(long long)(col0 + wave * CPW + q) * ldx + base + lane];
#pragma unroll
            for (int q = 0; q < HALO; ++q) {
                const int col = wave * CPW + q * 8 + hcol;
                pre[CPW + q] = (q * 8 + hcol < CPW) ? X[(long long)(col0 + col) * ldx + base + hrow] : 0.f;
            }
        } else {
#pragma unroll
            for (int q = 0; q < CPW; ++q) {
                const int col = col0 + wave * CPW + q;
                const long long r = base + lane;
                pre[q] = (col < batch && r >= 0 && r < n_in) ? X[(long long)col * ldx + r] : 0.f;
            }
#pragma unroll
            for (int q = 0; q < HALO; ++q) {
                const int col = col0 + wave * CPW + q * 8 + hcol;
                const long long r = base + hrow;
                pre[CPW + q] = (q * 8 + hcol < CPW && col < batch && r >= 0 && r < n_in)
                                   ? X[(long long)col * ldx + r] : 0.f;
            }
        }
    };
    auto commit = [&](float *buf) {
#pragma unroll
        for (int q = 0; q < CPW; ++q) buf[(wave * CPW + q) * SP_PITCH + lane] = pre[q];
#pragma unroll
        for (int q = 0; q < HALO; ++q)
            if (q * 8 + hcol < CPW) buf[(wave * CPW + q * 8 + hcol) * SP_PITCH + hrow] = pre[CPW + q];
    };

    issue(0);
    commit(lds[0]);
    __syncthreads();

    const long long arow = (long long)row0 + wave * T;
    for (int c = 0; c < nchunks; ++c) {
        const bool more = c + 1 < nchunks;
        if (more) issue(c + 1);

        const sc_chunk_ptr ck = cks + c;
        const int s0 = ck->s0;
        const int len = ck->len;
        const float *win_lds = &lds[c & 1][lane * SP_PITCH + wave * T];
        const long long base = (long long)row0 + s0;
        const bool interior = (base >= 0) & (base + SP_STAGED <= n_in) & (row0 + SP_ROWS <= n_out);
#define CUVDIA_SPMM_CASE(L)                                                                   \
        case L:                                                                               \
            if (interior) spmm_chunk<T, L, false>(acc, win_lds, svals, ck, s0, stride, arow, ashift, n_out, n_in); \
            else          spmm_chunk<T, L, true >(acc, win_lds, svals, ck, s0, stride, arow, ashift, n_out, n_in); \
            break;
        switch (len) {
            CUVDIA_SPMM_CASE(1) CUVDIA_SPMM_CASE(2) CUVDIA_SPMM_CASE(3) CUVDIA_SPMM_CASE(4)
            CUVDIA_SPMM_CASE(5) CUVDIA_SPMM_CASE(6) CUVDIA_SPMM_CASE(7) CUVDIA_SPMM_CASE(8)
            default: break;
        }
#undef CUVDIA_SPMM_CASE
        if (more) commit(lds[(c + 1) & 1]);
        __syncthreads();
    }

    // epilogue: lanes-along-columns -> lanes-along-rows through LDS
    float *out = &lds[0][0];
#pragma unroll
    for (int t = 0; t < T; ++t) out[lane * SP_OPITCH + wave * T + t] = acc[t];
    __syncthreads();
    const long long row = (long long)row0 + lane;
    if (row < n_out) {
#pragma unroll
        for (int q = 0; q < CPW; ++q) {
            const int col = wave * CPW + q;
            if (col0 + col < batch) {
                const float v = out[col * SP_OPITCH + lane];
                float *y = Y + (long long)(col0 + col) * ldy + row;
                *y = (beta == 0.f) ? alpha * v : beta * (*y) + alpha * v;
            }
        }
    }
}

// ------------------------------------------------------------ tiled dd2dia --
//
// Workgroup = 256 rows of ONE run chunk (<= 8 consecutive diagonals), 4 waves.
// Lane l owns rows row0 + 4l .. 4l+3 and 4 x len partial sums; wave q walks
// the batch-column groups g = q, q+4, ... (4 columns per group).  Per group
// the wave stages, privately (no workgroup barrier), rows
// [row0 + s0, row0 + s0 + 264) of B for the 4 columns into LDS with lanes
// along rows; each lane then reads its 4 + len - 1 wide window with 16-byte
// LDS reads, loads its 4 rows of A straight from global (16-byte, perfectly
// coalesced) and issues 4 x len FMAs per column.  The staging of the next
// group is issued before the FMAs of the current one.  The four waves'
// partial sums meet in LDS and are added in wave order.

constexpr int DD_ROWS = 256;
constexpr int DD_BG = 4;
constexpr int DD_STAGED = 264;     // 256 + CHUNK_MAX
constexpr int DD_PITCH = 264;

template <int LC>
__device__ __forceinline__ void dd2dia_tile(float *lds, sc_chunk_ptr ck, int row0,
                                            float *__restrict__ C, long long stride,
                                            const float *__restrict__ A, long long lda,
                                            const float *__restrict__ B, long long ldb,
                                            int h, int w, int batch, float alpha, float beta,
                                            int a_vec)
{
    constexpr int WIN = 4 + LC - 1;
    constexpr int WQ = (WIN + 3) / 4;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int s0 = ck->s0;
    const long long base = (long long)row0 + s0;
    const bool b_interior = (base >= 0) & (base + DD_STAGED <= w);
    const long long myrow = (long long)row0 + 4 * lane;
    const bool a_full = (myrow + 3 < h) & (a_vec != 0);

    float acc[4][LC];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int j = 0; j < LC; ++j) acc[t][j] = 0.f;

    float *mybuf = lds + wave * (2 * DD_BG * DD_PITCH);
    const int ngroups = (batch + DD_BG - 1) / DD_BG;
    float pre[DD_BG * 4 + 1];
    const int hb = lane >> 3, hrow = DD_ROWS + (lane & 7);

    auto issue = [&](int g) {
        const int b0 = g * DD_BG;
        if (b_interior && b0 + DD_BG <= batch) {
#pragma unroll
            for (int i = 0; i < DD_BG; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    pre[i * 4 + q] = B[(long long)(b0 + i) * ldb + base + q * 64 + lane];
            pre[DD_BG * 4] = (hb < DD_BG) ? B[(long long)(b0 + hb) * ldb + base + hrow] : 0.f;
        } else {
#pragma unroll
            for (int i = 0; i < DD_BG; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const long long r = base + q * 64 + lane;
                    pre[i * 4 + q] = (b0 + i < batch && r >= 0 && r < w)
                                         ? B[(long long)(b0 + i) * ldb + r] : 0.f;
                }
            const long long r = base + hrow;
            pre[DD_BG * 4] = (hb < DD_BG && b0 + hb < batch && r >= 0 && r < w)
                                 ? B[(long long)(b0 + hb) * ldb + r] : 0.f;
        }
    };
    auto commit = [&](float *buf) {
#pragma unroll
        for (int i = 0; i < DD_BG; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) buf[i * DD_PITCH + q * 64 + lane] = pre[i * 4 + q];
        if (hb < DD_BG) buf[hb * DD_PITCH + hrow] = pre[DD_BG * 4];
    };

    int g = wave;
    if (g < ngroups) { issue(g); commit(mybuf); }
    for (int it = 0; g < ngroups; g += 4, ++it) {
        float *cur = mybuf + (it & 1) * (DD_BG * DD_PITCH);
        float *nxt = mybuf + ((it + 1) & 1) * (DD_BG * DD_PITCH);
        const bool more = g + 4 < ngroups;
        if (more) issue(g + 4);
        wave_lds_fence();
#pragma unroll
        for (int i = 0; i < DD_BG; ++i) {
            const int b = g * DD_BG + i;
            float a[4] = {0.f, 0.f, 0.f, 0.f};
            if (b < batch) {
                const float *ap = A + (long long)b * lda + myrow;
                if (a_full) {
                    const float4 v = *reinterpret_cast<const float4 *>(ap);
                    a[0] = v.x; a[1] = v.y; a[2] = v.z; a[3] = v.w;
                } else {
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        if (myrow + t < h) a[t] = ap[t];
                }
            }
            float win[WQ * 4];
            const float4 *p4 = reinterpret_cast<const float4 *>(cur + i * DD_PITCH + 4 * lane);
#pragma unroll
            for (int q = 0; q < WQ; ++q) {
                const float4 v = p4[q];
                win[4 * q + 0] = v.x; win[4 * q + 1] = v.y; win[4 * q + 2] = v.z; win[4 * q + 3] = v.w;
            }
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int j = 0; j < LC; ++j)
                    acc[t][j] = __builtin_fmaf(a[t], win[t + j], acc[t][j]);
        }
        wave_lds_fence();
        if (more) commit(nxt);
    }

    // combine the four waves' partial sums in wave order
    __syncthreads();
    float *red = lds;                      // [wave][4*LC][64]
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int j = 0; j < LC; ++j)
            red[(wave * 32 + t * LC + j) * 64 + lane] = acc[t][j];
    __syncthreads();
    for (int j = wave; j < LC; j += 4) {
        float *cd = C + (long long)ck->slot[j] * stride;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int ai = (t * LC + j) * 64 + lane;
            const float total = ((red[ai] + red[32 * 64 + ai]) + red[2 * 32 * 64 + ai]) + red[3 * 32 * 64 + ai];
            const long long o = myrow + t;
            const long long in = o + s0 + j;
            if (o < h && in >= 0 && in < w)
                cd[o] = (beta == 0.f) ? alpha * total : beta * cd[o] + alpha * total;
        }
    }
}

__global__ __launch_bounds__(256) void dd2dia_tiled_kernel(
    const Chunk *__restrict__ chunks, int nchunks, float *__restrict__ C, int stride,
    const float *__restrict__ A, long long lda, const float *__restrict__ B, long long ldb,
    int h, int w, int batch, float alpha, float beta, int a_vec)
{
    __shared__ __attribute__((aligned(16))) float lds[4 * 2 * DD_BG * DD_PITCH];
    const int tile = xcd_tile(blockIdx.x, gridDim.x);
    const int rowtile = tile / nchunks;
    const sc_chunk_ptr ck = scalar_ptr(chunks) + (tile - rowtile * nchunks);
    const int row0 = rowtile * DD_ROWS;
#define CUVDIA_DD_CASE(L) \
    case L: dd2dia_tile<L>(lds, ck, row0, C, stride, A, lda, B, ldb, h, w, batch, alpha, beta, a_vec); break;
    switch (ck->len) {
        CUVDIA_DD_CASE(1) CUVDIA_DD_CASE(2) CUVDIA_DD_CASE(3) CUVDIA_DD_CASE(4)
        CUVDIA_DD_CASE(5) CUVDIA_DD_CASE(6) CUVDIA_DD_CASE(7) CUVDIA_DD_CASE(8)
        default: break;
    }
#undef CUVDIA_DD_CASE
}

}  // namespace

// ---------------------------------------------------------------- launchers --

hipError_t launch_spmm_generic(const DiaView &A, const float *vals, const float *B, long long ldb,
                               float *dst, long long ldd, int batch, bool trans,
                               float alpha, float beta, hipStream_t stream)
{
    const int n_out = trans ? A.w : A.h;
    constexpr int CB = 4;
    const unsigned gx = (unsigned)((n_out + 255) / 256);
    int done = 0;
    // grid.y is limited to 65535: walk very wide batches in slabs
    while (done < batch) {
        const int slab = batch - done < 65535 * CB ? batch - done : 65535 * CB;
        const dim3 grid(gx, (unsigned)((slab + CB - 1) / CB));
        hipLaunchKernelGGL(spmm_generic_kernel<CB>, grid, dim3(256), 0, stream,
                           A.offsets_dev, A.nd, vals, A.stride, A.h, A.w, A.rf,
                           B + (long long)done * ldb, ldb, dst + (long long)done * ldd, ldd,
                           n_out, slab, trans ? 1 : 0, alpha, beta);
        done += slab;
    }
    return hipGetLastError();
}

hipError_t launch_spmm_tiled(const DiaView &A, const float *vals, const float *B, long long ldb,
                             float *dst, long long ldd, int batch, bool trans,
                             float alpha, float beta, hipStream_t stream)
{
    const int n_out = trans ? A.w : A.h;
    const int n_in = trans ? A.h : A.w;
    const long long row_tiles = (n_out + SP_ROWS - 1) / SP_ROWS;
    const long long col_tiles = (batch + SP_COLS - 1) / SP_COLS;
    if (row_tiles * col_tiles > 0x7fffffffLL) return hipErrorInvalidValue;
    const Chunk *chunks = trans ? A.chunks_t_dev : A.chunks_n_dev;
    const int nchunks = trans ? A.n_chunks_t : A.n_chunks_n;
    constexpr int T = 16, WAVES = 4;
    hipLaunchKernelGGL((spmm_tiled_kernel<T, WAVES>), dim3((unsigned)(row_tiles * col_tiles)),
                       dim3(64 * WAVES), 0, stream, chunks, nchunks, vals, A.stride, trans ? 1 : 0,
                       B, ldb, dst, ldd, n_out, n_in, batch, alpha, beta, (int)col_tiles);
    return hipGetLastError();
}

hipError_t launch_dd2dia_generic(const DiaView &C, float *vals, const float *A, long long lda,
                                 const float *B, long long ldb, int batch,
                                 float alpha, float beta, hipStream_t stream)
{
    const unsigned gx = (unsigned)((C.h + 255) / 256);
    int done = 0;
    while (done < C.nd) {
        const int slab = C.nd - done < 65535 ? C.nd - done : 65535;
        hipLaunchKernelGGL(dd2dia_generic_kernel, dim3(gx, (unsigned)slab), dim3(256), 0, stream,
                           C.offsets_dev + done, vals + (long long)done * C.stride, C.stride,
                           C.h, C.w, C.rf, A, lda, B, ldb, batch, alpha, beta);
        done += slab;
    }
    return hipGetLastError();
}

hipError_t launch_dd2dia_tiled(const DiaView &C, float *vals, const float *A, long long lda,
                               const float *B, long long ldb, int batch,
                               float alpha, float beta, hipStream_t stream)
{
    const long long row_tiles = (C.h + DD_ROWS - 1) / DD_ROWS;
    const long long blocks = row_tiles * C.n_chunks_n;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    // 16-byte loads of A need an aligned base and leading dimension; row tiles
    // start at multiples of 256 and lanes at multiples of 4 rows.
    const int a_vec = (reinterpret_cast<unsigned long long>(A) % 16 == 0) && (lda % 4 == 0);
    hipLaunchKernelGGL(dd2dia_tiled_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                       C.chunks_n_dev, C.n_chunks_n, vals, C.stride, A, lda, B, ldb,
                       C.h, C.w, batch, alpha, beta, a_vec);
    return hipGetLastError();
}

}  // namespace cuvdia
