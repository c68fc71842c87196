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
//   spmm    acc = 0; for each run chunk in ascending shift order (a tile with
//           exactly one chunk whose rows cross an end of the dense operand
//           takes that chunk first), for each diagonal of the chunk in
//           ascending shift order:
//           acc = fma(a, x, acc); then dst = beta*dst + alpha*acc
//           (dst = alpha*acc when beta == 0, dst never read).
//           The generic kernel walks the offset table in table order instead.
//   dd2dia  a single chunk: four partial sums, wave q of the workgroup owning
//           batch columns {4*g + i : g = q (mod 4), i < 4} in ascending order,
//           each acc = fma(a, b, acc); total = ((p0 + p1) + p2) + p3.
//           A chunk pair: eight sums s_q over g = q (mod 8);
//           p_q = s_q + s_{q+4}, then total as above.
//           C = beta*C + alpha*total.  The generic kernel and the window-table
//           kernels sum the batch serially in ascending column order (the one
//           for window rows of at most 8 diagonals, on launches of few tiles,
//           as 2 or 4 ranges of the batch whose sums are added in range order).
#include <hip/hip_runtime.h>

#include <cstring>
#include <mutex>
#include <type_traits>

#include "kernels.hpp"

// This file is compiled seven times (CUVDIA_PART = 1 .. 7, see the Makefile), each translation unit
// instantiating one share of the kernel templates, so that the shares compile in parallel: parts 1 - 3 hold
// the tiled SpMM kernels by longest chunk (1 - 5, 6 - 9, 10 - 13), part 5 the walking SpMM kernels, part 6
// the window-table projection for window rows of at most 8 diagonals, part 7 the one for rows of 9 to 13, part 4
// everything else.  Without the macro one unit holds everything.
#ifndef CUVDIA_PART
#define CUVDIA_PART 0
#endif
#define CUVDIA_IN_PART(p) (CUVDIA_PART == 0 || CUVDIA_PART == (p))

namespace cuvdia {
namespace {

// Results leave through non-temporal stores: they are streamed past the
// caches instead of waiting there, dirty, for the write-back at the kernel's
// end, which every store of a one-round kernel would otherwise meet at once.
template <class V>
__device__ __forceinline__ void stream_store(V *p, V v)
{
    __builtin_nontemporal_store(v, p);
}
// Four consecutive floats as one 16-byte store; 4-byte alignment is all a 16-byte global store needs.
__device__ __forceinline__ void stream_store4(float *p, float a, float b, float c, float d)
{
    typedef float f4u __attribute__((ext_vector_type(4), aligned(4)));
    __builtin_nontemporal_store(f4u{a, b, c, d}, reinterpret_cast<f4u *>(p));
}

// Hardware hands consecutive workgroup ids to the 8 XCDs round-robin, and each
// XCD has its own L2.  Remap so that every XCD works on contiguous spans of
// tiles: neighbouring row tiles share dense-operand rows (the halo and the
// bands +-px apart), which then hit in that XCD's L2.  The tiles are dealt out
// in groups of 8 spans of XCD_SPAN, one span per XCD and group, so that work
// which varies along the rows (chunks falling outside the operand) still
// spreads evenly; the last, partial group is split into 8 near-equal spans.
// The very last span is dealt backwards: the tiles at the high end of the
// rows take the slower body for tiles at the operand's ends, exactly like the
// first tiles of the first span, and dealt in order they would be the last to
// start as well -- a launch of one or two rounds then ends when they do.
constexpr int XCD_SPAN = 64;
__device__ __forceinline__ int xcd_tile(int bid, int nblk)
{
    constexpr int XCDS = 8, GROUP = XCDS * XCD_SPAN;
    const int full = nblk / GROUP * GROUP;           // tiles in whole groups
    if (bid < full) {
        const int g = bid / GROUP, in = bid - g * GROUP;
        const int xcd = in % XCDS;
        int slot = in / XCDS;
        if (xcd == XCDS - 1 && (g + 1) * GROUP == nblk) slot = XCD_SPAN - 1 - slot;
        return g * GROUP + xcd * XCD_SPAN + slot;
    }
    const int rest = nblk - full, b = bid - full;
    const int q = rest / XCDS, r = rest % XCDS;
    const int xcd = b % XCDS;
    int slot = b / XCDS;
    if (xcd == XCDS - 1) slot = q - 1 - slot;        // the last span has q tiles (r < XCDS)
    return full + xcd * q + (xcd < r ? xcd : r) + slot;
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

// Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy
// as 1, 2, 3", SC'11): a counter-based generator, 4 x 32 random bits per
// 128-bit counter and 64-bit key, no state.  The result element (row, col)
// draws word col & 3 of the block with counter (row, col >> 2, 0, 0) and key
// (seed_lo, seed_hi), so a sample depends on the seed and the element's
// position only -- not on which kernel, tile or lane produced it.
struct SpRand4 { unsigned w[4]; };
__device__ __forceinline__ SpRand4 sp_philox(unsigned row, unsigned colblock, unsigned k0, unsigned k1)
{
    unsigned c0 = row, c1 = colblock, c2 = 0u, c3 = 0u;
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const unsigned hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
        const unsigned hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
        c0 = hi1 ^ c1 ^ k0;
        c1 = lo1;
        c2 = hi0 ^ c3 ^ k1;
        c3 = lo0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return SpRand4{{c0, c1, c2, c3}};
}
// 24 random bits -> a uniform variate in [0, 1), exactly representable
__device__ __forceinline__ float sp_uniform(unsigned word) { return (float)(word >> 8) * 0x1p-24f; }

// Last step of an SpMM result element: optional per-row bias, optional
// logistic sigmoid 1/(1+exp(-v)) (src/cuv/tensor_ops/functors.hpp:122),
// optional Bernoulli sample of that probability, v > u
// (src/cuv/random/random.cu:86-91).
__device__ __forceinline__ float sp_finish(float v, float bias, int act, unsigned word = 0u)
{
    v += bias;
    if (act == 0) return v;
    // v_exp_f32 and v_rcp_f32 (1 ulp each) instead of the library's exp and an
    // IEEE division: p is off by < 1e-7 absolute, inside what the sum's own
    // rounding allows, and the store costs a dozen instructions less per element
    const float p = __builtin_amdgcn_rcpf(1.f + __expf(-v));
    return act == 2 ? (p > sp_uniform(word) ? 1.f : 0.f) : p;
}

// ------------------------------------------------------------------ generic --

template <int CB>
__global__ __launch_bounds__(256) void spmm_generic_kernel(
    const int *__restrict__ offsets, int nd, const float *__restrict__ vals, int stride,
    int h, int w, int rf, const float *__restrict__ X, long long ldx,
    float *__restrict__ Y, long long ldy, int n_out, int batch, int trans,
    float alpha, float beta, SpEpilogue ep)
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
            const float v = (beta == 0.f) ? alpha * acc[c] : beta * (*y) + alpha * acc[c];
            const unsigned col = (unsigned)(c0 + c);
            const unsigned word = ep.act == 2 ? sp_philox((unsigned)o, col >> 2, ep.seed_lo, ep.seed_hi).w[col & 3u] : 0u;
            stream_store(y, sp_finish(v, ep.bias ? ep.bias[o] : 0.f, ep.act, word));
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

// Mean of every stored diagonal over its valid slots (row_fact == 1):
// dst[d] = sum_{n < N_d} vals[d*stride + i_start + n] / N_d
// (src/cuv/matrix_ops/diagonals.cu:24-51).  One workgroup of 1024 threads per
// diagonal.  Summation order: thread t keeps 8 running sums, sum u taking the
// elements n = 8192*k + 1024*u + t in ascending k; the thread adds them in
// ascending u; the 1024 thread sums are folded in LDS, s[t] += s[t + w] for
// w = 512, 256, .., 1.  A diagonal with no valid slot yields 0.
constexpr int AVG_THREADS = 1024;
__global__ __launch_bounds__(AVG_THREADS) void avg_diagonals_kernel(
    const int *__restrict__ offsets, const float *__restrict__ vals, int stride, int h, int w,
    float *__restrict__ dst)
{
    __shared__ float part[AVG_THREADS];
    const int d = blockIdx.x, t = threadIdx.x;
    const long long k = offsets[d];
    const long long i_start = k < 0 ? -k : 0, j_start = k > 0 ? k : 0;
    const long long N = min((long long)h - i_start, (long long)w - j_start);
    const float *x = vals + (long long)d * stride + i_start;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (long long base = 0; base < N; base += 8 * AVG_THREADS) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const long long n = base + AVG_THREADS * u + t;
            acc[u] += n < N ? x[n] : 0.f;
        }
    }
    float sum = acc[0];
#pragma unroll
    for (int u = 1; u < 8; ++u) sum += acc[u];
    part[t] = sum;
    __syncthreads();
    for (int wdt = AVG_THREADS / 2; wdt >= 1; wdt >>= 1) {
        if (t < wdt) part[t] += part[t + wdt];
        __syncthreads();
    }
    if (t == 0) dst[d] = N > 0 ? part[0] / (float)N : 0.f;
}

// W[i] = alpha*dW[i] + beta*W[i]: the weight update that follows the
// gradient (src/cuv/tensor_ops/rprop.cu:148-156).  Purely HBM-bound: 8 bytes
// read and 4 written per element, 16-byte accesses once both arrays are
// 16-byte aligned (the first elements up to that point, and the tail, go one
// by one).
constexpr int AXPBY_THREADS = 256;
__global__ __launch_bounds__(AXPBY_THREADS) void axpby_kernel(
    float *__restrict__ W, const float *__restrict__ dW, long long n, float alpha, float beta, int head, int vec)
{
    const long long tid = (long long)blockIdx.x * AXPBY_THREADS + threadIdx.x;
    const long long nthreads = (long long)gridDim.x * AXPBY_THREADS;
    if (!vec) {                                      // the arrays are misaligned against each other
        for (long long i = tid; i < n; i += nthreads) W[i] = alpha * dW[i] + beta * W[i];
        return;
    }
    // `head` (< 4) elements precede the first 16-byte boundary of both arrays
    const long long nvec = (n - head) / 4;
    float4 *W4 = reinterpret_cast<float4 *>(W + head);
    const float4 *D4 = reinterpret_cast<const float4 *>(dW + head);
    for (long long i = tid; i < nvec; i += nthreads) {
        const float4 d = D4[i];
        float4 w = W4[i];
        w.x = alpha * d.x + beta * w.x;
        w.y = alpha * d.y + beta * w.y;
        w.z = alpha * d.z + beta * w.z;
        w.w = alpha * d.w + beta * w.w;
        W4[i] = w;
    }
    const long long rest = n - head - 4 * nvec;      // < 4
    if (tid < head) W[tid] = alpha * dW[tid] + beta * W[tid];
    if (tid < rest) {
        const long long i = head + 4 * nvec + tid;
        W[i] = alpha * dW[i] + beta * W[i];
    }
}

// m = momentum_weight*m - lr*(dW + l2decay*W); W += m; M = m
// (src/cuv/tensor_ops/rprop.cu:158-170, the device kernel's formula).  Three
// arrays read, two written: 20 bytes per element, HBM-bound; same layout of
// the work as axpby_kernel.
__global__ __launch_bounds__(AXPBY_THREADS) void momentum_kernel(
    float *__restrict__ W, float *__restrict__ M, const float *__restrict__ dW, long long n,
    float lr, float mw, float l2, int head, int vec)
{
    const long long tid = (long long)blockIdx.x * AXPBY_THREADS + threadIdx.x;
    const long long nthreads = (long long)gridDim.x * AXPBY_THREADS;
    auto one = [&](long long i) {
        const float m = mw * M[i] - lr * (dW[i] + l2 * W[i]);
        W[i] += m;
        M[i] = m;
    };
    if (!vec) {
        for (long long i = tid; i < n; i += nthreads) one(i);
        return;
    }
    const long long nvec = (n - head) / 4;
    float4 *W4 = reinterpret_cast<float4 *>(W + head);
    float4 *M4 = reinterpret_cast<float4 *>(M + head);
    const float4 *D4 = reinterpret_cast<const float4 *>(dW + head);
    for (long long i = tid; i < nvec; i += nthreads) {
        const float4 d = D4[i];
        float4 w = W4[i], m = M4[i];
        m.x = mw * m.x - lr * (d.x + l2 * w.x); w.x += m.x;
        m.y = mw * m.y - lr * (d.y + l2 * w.y); w.y += m.y;
        m.z = mw * m.z - lr * (d.z + l2 * w.z); w.z += m.z;
        m.w = mw * m.w - lr * (d.w + l2 * w.w); w.w += m.w;
        W4[i] = w;
        M4[i] = m;
    }
    const long long rest = n - head - 4 * nvec;      // < 4
    if (tid < head) one(tid);
    if (tid < rest) one(head + 4 * nvec + tid);
}

// -------------------------------------------------------------- tiled spmm --
//
// Workgroup = 64 output rows x 64 batch columns, 8 waves of T = 8 rows each.
// Lane l of every wave owns batch column col0 + l and T running sums.  Per
// run chunk (<= 13 consecutive shifts starting at s0):
//   1. the dense rows a0 .., a0 = row0 + s0, that the chunk touches are staged
//      in LDS for the 64 columns, LDS row i of a column holding dense row
//      a0 + i, together with the chunk's diagonals for the 64 rows (wave w
//      fetches diagonal w, one 256-byte row segment).  Rows outside the
//      operand and diagonal slots outside the matrix become zeros (an
//      out-of-range buffer offset reads as 0), so the arithmetic below needs
//      no guards and never sees padding;
//   2. each lane reads its column's window of T + LCK - 1 values with 16-byte
//      LDS reads (the column pitch / 4 is odd, so the 64 lanes spread over
//      all banks).  The kernel is instantiated for LCK = the longest chunk
//      of the table; a chunk of LCK diagonals runs one straight-line block
//      of FMAs, a shorter one only the diagonals it has (a wave-uniform test
//      per diagonal), so no dense value meets a diagonal that is not stored;
//   3. for each diagonal j the wave reads A_j[its T rows] into one VGPR (lane
//      & (T-1) selects the row) and issues T FMAs whose first operand is that
//      VGPR broadcast within each 16-lane row by DPP (row_newbcast:t):
//          acc[t] = fma(A_j[row t], win[t + j], acc[t]).
// There are two bodies.  Tiles all of whose rows exist and none of whose
// chunks straddles an end of the dense operand -- all but a few of a large
// matrix -- take the lean body (spmm_tile_lean): its loads write LDS directly,
// so staging costs the waves 4 instructions per chunk.  The tiles at the
// operand's ends take spmm_tile_edge, which stages through registers because
// it has to clamp and shift what it fetches.  Both are software-pipelined
// three chunks deep and transpose the sums through LDS at the end so that the
// store to dst runs along the rows; the lean body reads the chunk table
// through scalar loads, the edge body keeps it in vector registers (lane i
// <-> entry i, read with v_readlane).

constexpr int SP_ROWS = 64;        // output rows per workgroup
constexpr int SP_COLS = 64;        // batch columns per workgroup (one per lane)
constexpr int SP_QUADS = 20;       // 16-byte pieces staged per column (80 rows)
constexpr int SP_CPI = 3;          // columns per load instruction (3 x 20 lanes)
constexpr int SP_GROUPS = (SP_COLS + SP_CPI - 1) / SP_CPI;             // 22 column groups
constexpr int SP_PITCH = 84;       // floats between staged columns
constexpr int SP_OPITCH = 68;      // floats between columns in the epilogue
constexpr int SP_XFLOATS = SP_COLS * SP_PITCH;
constexpr int SP_ADIAGS = 16;      // diagonals a chunk's LDS block has room for (>= SP_CHUNK_MAX)
constexpr int SP_AVALS = SP_ADIAGS * SP_ROWS;   // diagonal values per workgroup per chunk
constexpr int SP_DUMP = SP_XFLOATS + SP_AVALS;  // where idle lanes write
constexpr int SP_STAGE_FLOATS = SP_DUMP + 4;
constexpr int SP_WALK_WGS = 512;       // workgroups a walking launch aims at (two per CU)
constexpr int SP_RENUMBER_MIN_TILES = 1024;   // launches of more than two rounds renumber the row tiles of a window table
constexpr int SP_WALK_MIN_WGS = 384;   // below this the chip is not filled: the tile-by-tile kernels serve
constexpr int SP_MAX_CHUNKS = 256;   // chunk-table entries a wave can keep in registers (4 sets of 64)

// Per-wave shape: T rows (8 or 16, at most one DPP row of 16 lanes), so a
// workgroup has 64 / T waves.
template <int T>
struct SpShape {
    static_assert(T == 8 || T == 16, "rows per wave");
    static constexpr int WAVES = SP_ROWS / T;
    static constexpr int LOADS = (SP_GROUPS + WAVES - 1) / WAVES;      // 16-byte loads per wave per chunk
    static constexpr int CPW = SP_COLS / WAVES;                        // columns each wave stores in the epilogue
};

// APW: diagonals each wave fetches per chunk, ceil(LCK / waves)
template <int T, int APW>
struct SpStage {
    float4 x[SpShape<T>::LOADS];
    float a[APW];
    int shift;              // rows the pieces were fetched away from their place (0 except at the operand's ends)
    bool edge;              // some staged row does not exist (wave-uniform)
};

// One chunk-table entry as a wave needs it: shift, length, and the table
// positions of the diagonals this wave fetches.
template <int APW>
struct SpInfo {
    int s0, len;
    int slot[APW];
};

template <int LCK, int T>
struct SpWindow {
    static constexpr int WQ = (T + LCK - 1 + 3) / 4;
    float w[WQ * 4];
    float a[LCK];
};

// acc[T0 + t] += bcast_{T0 + t}(a) * win[J + T0 + t], t = 0..7: eight FMAs whose
// first operand is lane T0 + t of each 16-lane row of `a` (DPP row_newbcast).
// A DPP operand must not have been written by a VALU instruction in the two
// preceding issue slots; the leading s_nop covers whatever the compiler
// placed before the block.
template <int J, int T0, int NA, int NW>
__device__ __forceinline__ void fma_block8(float (&acc)[NA], float a, const float (&win)[NW])
{
    asm("s_nop 1\n\t"
        "v_fmac_f32_dpp %0, %8, %9 row_newbcast:%17 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %1, %8, %10 row_newbcast:%18 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %2, %8, %11 row_newbcast:%19 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %3, %8, %12 row_newbcast:%20 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %4, %8, %13 row_newbcast:%21 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %5, %8, %14 row_newbcast:%22 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %6, %8, %15 row_newbcast:%23 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %7, %8, %16 row_newbcast:%24 row_mask:0xf bank_mask:0xf"
        : "+v"(acc[T0 + 0]), "+v"(acc[T0 + 1]), "+v"(acc[T0 + 2]), "+v"(acc[T0 + 3]),
          "+v"(acc[T0 + 4]), "+v"(acc[T0 + 5]), "+v"(acc[T0 + 6]), "+v"(acc[T0 + 7])
        : "v"(a), "v"(win[J + T0 + 0]), "v"(win[J + T0 + 1]), "v"(win[J + T0 + 2]), "v"(win[J + T0 + 3]),
          "v"(win[J + T0 + 4]), "v"(win[J + T0 + 5]), "v"(win[J + T0 + 6]), "v"(win[J + T0 + 7]),
          "n"(T0 + 0), "n"(T0 + 1), "n"(T0 + 2), "n"(T0 + 3), "n"(T0 + 4), "n"(T0 + 5), "n"(T0 + 6), "n"(T0 + 7));
}

template <int LCK, int T, int J>
__device__ __forceinline__ void spmm_rows(float (&acc)[T], const SpWindow<LCK, T> &win)
{
    if constexpr (J < LCK) {
        fma_block8<J, 0>(acc, win.a[J], win.w);
        if constexpr (T == 16) fma_block8<J, 8>(acc, win.a[J], win.w);
        spmm_rows<LCK, T, J + 1>(acc, win);
    }
}

// The FMAs of N consecutive diagonals J0 .. J0+N-1 of a chunk for a wave of 8 rows, as ONE statement:
// acc[t] += bcast_t(a[j]) * win[W0 + j + t].  A DPP operand must not have been written by a VALU instruction in
// the two preceding issue slots; inside the statement no FMA writes another's DPP operand (the a[j] come from
// LDS reads), so one leading s_nop -- for whatever the compiler placed before the statement -- serves all 8*N.
template <int J0, int N, int W0, int NA, int NW>
__device__ __forceinline__ void fma_diagonals8(float (&acc)[8], const float (&a)[NA], const float (&win)[NW])
{
    static_assert(N >= 1 && N <= 4 && J0 + N <= NA && W0 + J0 + N + 7 <= NW, "one statement takes at most 30 operands");
    if constexpr (N == 1) {
        asm("s_nop 1\n\t"
            "v_fmac_f32_dpp %0, %8, %9 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %1, %8, %10 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %2, %8, %11 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %3, %8, %12 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %4, %8, %13 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %5, %8, %14 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %6, %8, %15 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %7, %8, %16 row_newbcast:7 row_mask:0xf bank_mask:0xf"
            : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]), "+v"(acc[5]), "+v"(acc[6]), "+v"(acc[7])
            : "v"(a[J0 + 0]), "v"(win[W0 + J0 + 0]), "v"(win[W0 + J0 + 1]), "v"(win[W0 + J0 + 2]), "v"(win[W0 + J0 + 3]), "v"(win[W0 + J0 + 4]), "v"(win[W0 + J0 + 5]), "v"(win[W0 + J0 + 6]), "v"(win[W0 + J0 + 7]));
    }     else if constexpr (N == 2) {
        asm("s_nop 1\n\t"
            "v_fmac_f32_dpp %0, %8, %10 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %1, %8, %11 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %2, %8, %12 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %3, %8, %13 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %4, %8, %14 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %5, %8, %15 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %6, %8, %16 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %7, %8, %17 row_newbcast:7 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %0, %9, %11 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %1, %9, %12 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %2, %9, %13 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %3, %9, %14 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %4, %9, %15 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %5, %9, %16 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %6, %9, %17 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %7, %9, %18 row_newbcast:7 row_mask:0xf bank_mask:0xf"
            : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]), "+v"(acc[5]), "+v"(acc[6]), "+v"(acc[7])
            : "v"(a[J0 + 0]), "v"(a[J0 + 1]), "v"(win[W0 + J0 + 0]), "v"(win[W0 + J0 + 1]), "v"(win[W0 + J0 + 2]), "v"(win[W0 + J0 + 3]), "v"(win[W0 + J0 + 4]), "v"(win[W0 + J0 + 5]), "v"(win[W0 + J0 + 6]), "v"(win[W0 + J0 + 7]), "v"(win[W0 + J0 + 8]));
    }     else if constexpr (N == 3) {
        asm("s_nop 1\n\t"
            "v_fmac_f32_dpp %0, %8, %11 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %1, %8, %12 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %2, %8, %13 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %3, %8, %14 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %4, %8, %15 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %5, %8, %16 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %6, %8, %17 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %7, %8, %18 row_newbcast:7 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %0, %9, %12 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %1, %9, %13 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %2, %9, %14 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %3, %9, %15 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %4, %9, %16 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %5, %9, %17 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %6, %9, %18 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %7, %9, %19 row_newbcast:7 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %0, %10, %13 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %1, %10, %14 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %2, %10, %15 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %3, %10, %16 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %4, %10, %17 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %5, %10, %18 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %6, %10, %19 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %7, %10, %20 row_newbcast:7 row_mask:0xf bank_mask:0xf"
            : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]), "+v"(acc[5]), "+v"(acc[6]), "+v"(acc[7])
            : "v"(a[J0 + 0]), "v"(a[J0 + 1]), "v"(a[J0 + 2]), "v"(win[W0 + J0 + 0]), "v"(win[W0 + J0 + 1]), "v"(win[W0 + J0 + 2]), "v"(win[W0 + J0 + 3]), "v"(win[W0 + J0 + 4]), "v"(win[W0 + J0 + 5]), "v"(win[W0 + J0 + 6]), "v"(win[W0 + J0 + 7]), "v"(win[W0 + J0 + 8]), "v"(win[W0 + J0 + 9]));
    }     else if constexpr (N == 4) {
        asm("s_nop 1\n\t"
            "v_fmac_f32_dpp %0, %8, %12 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %1, %8, %13 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %2, %8, %14 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %3, %8, %15 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %4, %8, %16 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %5, %8, %17 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %6, %8, %18 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %7, %8, %19 row_newbcast:7 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %0, %9, %13 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %1, %9, %14 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %2, %9, %15 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %3, %9, %16 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %4, %9, %17 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %5, %9, %18 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %6, %9, %19 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %7, %9, %20 row_newbcast:7 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %0, %10, %14 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %1, %10, %15 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %2, %10, %16 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %3, %10, %17 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %4, %10, %18 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %5, %10, %19 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %6, %10, %20 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %7, %10, %21 row_newbcast:7 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %0, %11, %15 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %1, %11, %16 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %2, %11, %17 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %3, %11, %18 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %4, %11, %19 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %5, %11, %20 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %6, %11, %21 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %7, %11, %22 row_newbcast:7 row_mask:0xf bank_mask:0xf"
            : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]), "+v"(acc[5]), "+v"(acc[6]), "+v"(acc[7])
            : "v"(a[J0 + 0]), "v"(a[J0 + 1]), "v"(a[J0 + 2]), "v"(a[J0 + 3]), "v"(win[W0 + J0 + 0]), "v"(win[W0 + J0 + 1]), "v"(win[W0 + J0 + 2]), "v"(win[W0 + J0 + 3]), "v"(win[W0 + J0 + 4]), "v"(win[W0 + J0 + 5]), "v"(win[W0 + J0 + 6]), "v"(win[W0 + J0 + 7]), "v"(win[W0 + J0 + 8]), "v"(win[W0 + J0 + 9]), "v"(win[W0 + J0 + 10]));
    }
}

// the diagonals J .. J1 - 1 of a chunk (waves of 8 rows take them four to a statement)
template <int LCK, int T, int J, int J1>
__device__ __forceinline__ void spmm_rows_range(float (&acc)[T], const SpWindow<LCK, T> &win)
{
    if constexpr (J < J1) {
        if constexpr (T == 8) {
            constexpr int N = J1 - J < 4 ? J1 - J : 4;
            fma_diagonals8<J, N, 0>(acc, win.a, win.w);
            spmm_rows_range<LCK, T, J + N, J1>(acc, win);
        } else {
            fma_block8<J, 0>(acc, win.a[J], win.w);
            fma_block8<J, 8>(acc, win.a[J], win.w);
            spmm_rows_range<LCK, T, J + 1, J1>(acc, win);
        }
    }
}

// The same for a chunk of `len` < LCK diagonals (wave-uniform): the diagonals it does not have are skipped, not
// multiplied as zeros -- a product 0 * Inf or 0 * NaN with a dense row that the chunk's own diagonals do not
// reach would put a NaN where the reference's loop over stored elements leaves a finite sum.
template <int LCK, int T, int J, int J1>
__device__ __forceinline__ void spmm_rows_range_upto(float (&acc)[T], const SpWindow<LCK, T> &win, int len)
{
    if constexpr (J < J1) {
        if (J < len) {
            if constexpr (T == 8) {
                fma_diagonals8<J, 1, 0>(acc, win.a, win.w);
            } else {
                fma_block8<J, 0>(acc, win.a[J], win.w);
                fma_block8<J, 8>(acc, win.a[J], win.w);
            }
        }
        spmm_rows_range_upto<LCK, T, J + 1, J1>(acc, win, len);
    }
}
// diagonals J .. J1 - 1 of a chunk of `len` diagonals.  MIXED = false: the kernel for tables all of whose chunks
// have LCK diagonals (every window table): the straight-line block, no test.  MIXED = true: the guarded block for
// every chunk, full ones included (a second, straight-line copy for those made the variants for LCK >= 10 spill
// up to 60 registers; the tests are 2 scalar instructions per diagonal).
template <int LCK, int T, int J, int J1, bool MIXED>
__device__ __forceinline__ void spmm_rows_chunk(float (&acc)[T], const SpWindow<LCK, T> &win, int len)
{
    if constexpr (LCK == 1 || !MIXED) {
        spmm_rows_range<LCK, T, J, J1>(acc, win);
    } else {
        spmm_rows_range_upto<LCK, T, J, J1>(acc, win, len);
    }
}

template <int LCK, int T>
__device__ __forceinline__ void spmm_read_window(SpWindow<LCK, T> &win, const float *win_lds,
                                                 const float *a_lds)
{
    const float4 *p4 = reinterpret_cast<const float4 *>(win_lds);
#pragma unroll
    for (int q = 0; q < SpWindow<LCK, T>::WQ; ++q) {
        const float4 v = p4[q];
        win.w[4 * q + 0] = v.x; win.w[4 * q + 1] = v.y; win.w[4 * q + 2] = v.z; win.w[4 * q + 3] = v.w;
    }
#pragma unroll
    for (int j = 0; j < LCK; ++j) win.a[j] = a_lds[j * SP_ROWS];
}

// Buffer resource over [base, base + bytes): loads take a 32-bit VGPR byte
// offset, and an offset at or beyond `bytes` makes the hardware return 0
// instead of touching memory -- which is how rows before the operand, rows
// past its end and diagonal slots outside the matrix become zeros without a
// compare-and-select per load.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, unsigned bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, 0x00020000);
}
__device__ __forceinline__ float buffer_load_f32(__amdgpu_buffer_rsrc_t r, unsigned voff)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, 0, 0));
}
__device__ __forceinline__ float4 buffer_load_f32x4(__amdgpu_buffer_rsrc_t r, unsigned voff)
{
    return __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 0));
}
constexpr unsigned OOB_OFFSET = 0x80000000u;     // >= every resource size used here

// The body for tiles at the operand's ends.  The dense rows [a0, a0 + 80) of
// the 64 columns are fetched with 16-byte buffer loads into registers (20
// lanes per column and 3 columns per instruction) and written to LDS with
// 16-byte stores, columns 84 floats apart; a piece that straddles the
// operand's first or last row is fetched from the nearest in-range position
// and shifted into place on the way.  While the FMAs of chunk c run, chunk
// c+1 is being written to the other LDS buffer (its window is read right after
// the barrier), chunk c+2 is in flight and chunk c+3 has just been requested.
template <int LCK, int T, int NTAB, bool EP, bool MIXED>
__device__ __forceinline__ void spmm_tile_edge(
    float (&lds)[2][SP_STAGE_FLOATS], int row0, int col0,
    const Chunk *__restrict__ chunks, int nchunks, const float *__restrict__ vals, int stride,
    int ashift, const float *__restrict__ X, long long ldx, float *__restrict__ Y, long long ldy,
    int n_out, int n_in, int batch, float alpha, float beta, unsigned a_bytes, SpEpilogue ep)
{
    typedef SpShape<T> S;
    constexpr int SP_WAVES = S::WAVES, SP_LOADS = S::LOADS, SP_APW = (LCK + S::WAVES - 1) / S::WAVES, SP_CPW = S::CPW, SP_T = T;
    typedef SpStage<T, SP_APW> Stage;
    typedef SpInfo<SP_APW> Info;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    float acc[SP_T];
#pragma unroll
    for (int t = 0; t < SP_T; ++t) acc[t] = 0.f;

    // dense operand: resource from this tile's first column to the end of the
    // last valid column, so nothing outside the operand is ever touched.
    // Columns past the batch are replaced by the last valid one (their sums
    // are never stored).
    const int cols_here = min(SP_COLS, batch - col0);
    const unsigned x_bytes = (unsigned)(((long long)(cols_here - 1) * ldx + n_in) * 4);
    const __amdgpu_buffer_rsrc_t xr = make_rsrc(X + (long long)col0 * ldx, x_bytes);

    // beta != 0: the destination values this lane will combine at the end are
    // requested now, so their trip from memory overlaps the whole product.
    float ypre[SP_CPW];
    {
        const long long row = (long long)row0 + lane;
        const __amdgpu_buffer_rsrc_t yr = make_rsrc(
            Y + (long long)col0 * ldy, beta != 0.f ? (unsigned)(((long long)(cols_here - 1) * ldy + n_out) * 4) : 0u);
#pragma unroll
        for (int q = 0; q < SP_CPW; ++q) {
            const int col = wave * SP_CPW + q;
            ypre[q] = buffer_load_f32(yr, (row < n_out && col < cols_here)
                                              ? (unsigned)(col * ldy + row) * 4u : OOB_OFFSET);
        }
    }
    const int grp = lane / SP_QUADS;               // column within the instruction's group (3: idle lane)
    const int quad = lane - grp * SP_QUADS;        // 16-byte piece within the column
    unsigned col_off[SP_LOADS];                    // byte offset of this lane's column per load
    int lds_at[SP_LOADS];                          // float index in the stage buffer it is written to
#pragma unroll
    for (int it = 0; it < SP_LOADS; ++it) {
        const int col = (wave + SP_WAVES * it) * SP_CPI + grp;
        const bool live = (grp < SP_CPI) & (col < SP_COLS);
        col_off[it] = live ? (unsigned)min(col, cols_here - 1) * ((unsigned)ldx * 4u) : OOB_OFFSET;
        lds_at[it] = live ? col * SP_PITCH + 4 * quad : SP_DUMP;
    }
    // diagonal values: wave w fetches diagonals w, w + WAVES, ... of the chunk
    // for the workgroup's 64 rows
    const __amdgpu_buffer_rsrc_t ar = make_rsrc(vals, a_bytes);
    const int arow = row0 + lane;

    // The chunk table lives in vector registers, lane i of set k holding what
    // this wave needs of entry 64*k + i (shift, length, and the table position
    // of the diagonals it fetches); an entry is read with v_readlane into
    // scalar registers.  Nothing in the loop waits on memory for it.
    int tab_s0[NTAB], tab_len[NTAB], tab_slot[NTAB][SP_APW];
#pragma unroll
    for (int k = 0; k < NTAB; ++k) {
        const int *e = reinterpret_cast<const int *>(chunks + min(64 * k + lane, nchunks - 1));
        tab_s0[k] = e[0];
        tab_len[k] = e[1];
#pragma unroll
        for (int q = 0; q < SP_APW; ++q) tab_slot[k][q] = wave + SP_WAVES * q < CHUNK_SLOTS ? e[2 + wave + SP_WAVES * q] : -1;
    }
    auto fetch_info = [&](int c, Info &info) {
        const int cc = min(c, nchunks - 1);
        const int l = cc & 63;
        info.s0 = __builtin_amdgcn_readlane(tab_s0[0], l);
        info.len = __builtin_amdgcn_readlane(tab_len[0], l);
#pragma unroll
        for (int q = 0; q < SP_APW; ++q) info.slot[q] = __builtin_amdgcn_readlane(tab_slot[0][q], l);
#pragma unroll
        for (int k = 1; k < NTAB; ++k) {
            const bool here = (cc >> 6) == k;
            const int s0 = __builtin_amdgcn_readlane(tab_s0[k], l), len = __builtin_amdgcn_readlane(tab_len[k], l);
            info.s0 = here ? s0 : info.s0;
            info.len = here ? len : info.len;
#pragma unroll
            for (int q = 0; q < SP_APW; ++q) {
                const int sl = __builtin_amdgcn_readlane(tab_slot[k][q], l);
                info.slot[q] = here ? sl : info.slot[q];
            }
        }
    };

    auto chunk_len = [&](int c) {
        const int cc = min(c, nchunks - 1);
        int len = __builtin_amdgcn_readlane(tab_len[0], cc & 63);
#pragma unroll
        for (int k = 1; k < NTAB; ++k) {
            const int l = __builtin_amdgcn_readlane(tab_len[k], cc & 63);
            len = (cc >> 6) == k ? l : len;
        }
        return len;
    };

    // Dense rows come as 16-byte pieces.  A piece that straddles the operand's
    // first or last row is fetched from the nearest in-range position instead
    // (rows rc..rc+3) and shifted into place when it is written to LDS, so the
    // loads themselves never branch.
    auto issue = [&](const Info &info, Stage &st, int c) {
        const int s0 = info.s0;
        const int a0 = row0 + s0;
        const int r = a0 + 4 * quad;                       // first dense row of this lane's piece
        const int rc = min(max(r, 0), n_in - 4);
        const bool any = (r > -4) & (r < n_in);            // at least one row of the piece exists
        const unsigned row_off = (unsigned)rc * 4u;
#pragma unroll
        for (int it = 0; it < SP_LOADS; ++it)
            st.x[it] = buffer_load_f32x4(xr, (any & (col_off[it] != OOB_OFFSET)) ? col_off[it] + row_off : OOB_OFFSET);
        st.shift = rc - r;                                 // 0 except at the operand's ends
        st.edge = (a0 < 0) | (a0 + 4 * SP_QUADS > n_in);   // wave-uniform
#pragma unroll
        for (int q = 0; q < SP_APW; ++q) {
            const int j = wave + SP_WAVES * q;
            const int sl = info.slot[q];
            const int in = arow + s0 + j;                  // dense row this value multiplies
            const int vrow = ashift ? in : arow;           // row of the value inside its diagonal
            const bool ok = (j < info.len) & (sl >= 0) & (arow < n_out) & (in >= 0) & (in < n_in);
            const unsigned off = ((unsigned)sl * (unsigned)stride + (unsigned)vrow) * 4u;
            st.a[q] = buffer_load_f32(ar, ok ? off : OOB_OFFSET);
        }
    };
    auto commit = [&](const Stage &st, float *buf) {
        if (!st.edge) {
#pragma unroll
            for (int it = 0; it < SP_LOADS; ++it)
                *reinterpret_cast<float4 *>(buf + lds_at[it]) = st.x[it];
        } else {
            // out[k] = in[k - shift] where that exists, else 0
            const int d = st.shift;
#pragma unroll
            for (int it = 0; it < SP_LOADS; ++it) {
                const float v[4] = {st.x[it].x, st.x[it].y, st.x[it].z, st.x[it].w};
                float o[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    float t = 0.f;
#pragma unroll
                    for (int m = 0; m < 4; ++m) t = (k - d == m) ? v[m] : t;
                    o[k] = t;
                }
                *reinterpret_cast<float4 *>(buf + lds_at[it]) = make_float4(o[0], o[1], o[2], o[3]);
            }
        }
#pragma unroll
        for (int q = 0; q < SP_APW; ++q)
            buf[SP_XFLOATS + (wave + SP_WAVES * q) * SP_ROWS + lane] = st.a[q];
    };
    auto read_window = [&](SpWindow<LCK, T> &win, const float *buf) {
        spmm_read_window<LCK, T>(win, buf + lane * SP_PITCH + wave * SP_T,
                                 buf + SP_XFLOATS + wave * SP_T + (lane & (SP_T - 1)));
    };
    // Chunk k travels through stage set k & 1, LDS buffer k & 1, window set
    // k & 1 and table-entry set k & 1.  Entering iteration c: window(c) is in
    // registers, chunk c+1 has landed (or is landing) in `next`, chunk c+2 is
    // in flight in the other stage set, `info` holds table entry c+3.
    // Nothing in an iteration is conditional: past the end of the table the
    // last chunk is staged again (and never used), so the number of loads in
    // flight is the same on every path and each wait counts exactly.
    auto iteration = [&](int c, Stage &next, SpWindow<LCK, T> &win_cur, SpWindow<LCK, T> &win_next,
                         Info &info, Info &info_next) {
        commit(next, lds[(c + 1) & 1]);
        fetch_info(c + 4, info_next);
        issue(info, next, c + 3);
        spmm_rows_chunk<LCK, T, 0, LCK, MIXED>(acc, win_cur, MIXED ? chunk_len(c) : LCK);
        __syncthreads();
        read_window(win_next, lds[(c + 1) & 1]);
    };

    Stage st0, st1;
    SpWindow<LCK, T> w0, w1;
    Info i0, i1;
    fetch_info(0, i0);
    fetch_info(1, i1);
    issue(i0, st0, 0);
    fetch_info(2, i0);
    issue(i1, st1, 1);
    fetch_info(3, i1);
    commit(st0, lds[0]);
    issue(i0, st0, 2);
    __syncthreads();
    read_window(w0, lds[0]);
    int c = 0;
    if (nchunks & 1) {
        // odd table: one chunk alone first, then the register sets trade
        // places so the paired loop below starts in its usual state
        iteration(0, st1, w0, w1, i1, i0);
        { const Stage t = st0; st0 = st1; st1 = t; }
        { const SpWindow<LCK, T> t = w0; w0 = w1; w1 = t; }
        { const Info t = i0; i0 = i1; i1 = t; }
        c = 1;
    }
    for (; c < nchunks; c += 2) {
        iteration(c, st1, w0, w1, i1, i0);
        iteration(c + 1, st0, w1, w0, i0, i1);
    }

    // epilogue: lanes-along-columns -> lanes-along-rows through LDS (every
    // wave is past the last barrier, and the last window read came from the
    // other buffer or has completed)
    __syncthreads();
    float *out = &lds[0][0];
#pragma unroll
    for (int t = 0; t < SP_T; ++t) out[lane * SP_OPITCH + wave * SP_T + t] = acc[t];
    __syncthreads();
    const long long row = (long long)row0 + lane;
    if (row < n_out) {
        const float bias = (EP && ep.bias) ? ep.bias[row] : 0.f;
        float v[SP_CPW];
#pragma unroll
        for (int q = 0; q < SP_CPW; ++q) v[q] = out[(wave * SP_CPW + q) * SP_OPITCH + lane];   // all reads before the first store
        // the lane's 8 columns are two aligned blocks of 4: two generator calls
        SpRand4 rnd[SP_CPW / 4] = {};
        if (EP && ep.act == 2) {
#pragma unroll
            for (int k = 0; k < SP_CPW / 4; ++k)
                rnd[k] = sp_philox((unsigned)row, (unsigned)(col0 + wave * SP_CPW) / 4u + k, ep.seed_lo, ep.seed_hi);
        }
#pragma unroll
        for (int q = 0; q < SP_CPW; ++q) {
            const int col = wave * SP_CPW + q;
            if (col0 + col < batch) {
                float *y = Y + (long long)(col0 + col) * ldy + row;
                const float r = (beta == 0.f) ? alpha * v[q] : beta * ypre[q] + alpha * v[q];
                stream_store(y, EP ? sp_finish(r, bias, ep.act, rnd[q / 4].w[q & 3]) : r);
            }
        }
    }
}

// Loads that deliver straight into LDS (no vector register in between): lane i
// of the wave writes its 16 bytes at lds_byte_addr + 16*i; an
// out-of-range lane writes zeros, an inactive lane writes nothing.  They are
// vector-memory operations and complete in order with the wave's other loads
// (s_waitcnt vmcnt).  Written in assembly so that the waits below can be
// placed by hand: the loop keeps two chunks of them in flight across
// barriers, which no automatic placement allows.  M0 is written inside the
// statement without appearing among its clobbers: the compiler treats M0 as a
// reserved register (it never keeps a value there across other code, and sets
// it immediately before each instruction of its own that reads it), and it
// rejects reserved registers in a clobber list with a warning.
typedef int sp_int4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ sp_int4 raw_rsrc(const void *base, unsigned bytes)
{
    const unsigned long long b = reinterpret_cast<unsigned long long>(base);
    return sp_int4{(int)(unsigned)b, (int)((unsigned)(b >> 32) & 0xffffu), (int)bytes, 0x00020000};
}
__device__ __forceinline__ void lds_load_b128(sp_int4 rsrc, unsigned lds_byte_addr, unsigned voff, unsigned soff)
{
    // all three are wave-uniform by construction; this keeps them in scalar registers whatever the compiler infers
    lds_byte_addr = __builtin_amdgcn_readfirstlane(lds_byte_addr);
    soff = __builtin_amdgcn_readfirstlane(soff);
    rsrc = sp_int4{__builtin_amdgcn_readfirstlane(rsrc.x), __builtin_amdgcn_readfirstlane(rsrc.y),
                   __builtin_amdgcn_readfirstlane(rsrc.z), __builtin_amdgcn_readfirstlane(rsrc.w)};
    asm volatile("s_mov_b32 m0, %0\n\t"
                 "s_nop 0\n\t"
                 "buffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_byte_addr), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
// the same with 4 bytes per lane: lane i writes at lds_byte_addr + 4*i
__device__ __forceinline__ void lds_load_b32(sp_int4 rsrc, unsigned lds_byte_addr, unsigned voff)
{
    lds_byte_addr = __builtin_amdgcn_readfirstlane(lds_byte_addr);
    rsrc = sp_int4{__builtin_amdgcn_readfirstlane(rsrc.x), __builtin_amdgcn_readfirstlane(rsrc.y),
                   __builtin_amdgcn_readfirstlane(rsrc.z), __builtin_amdgcn_readfirstlane(rsrc.w)};
    asm volatile("s_mov_b32 m0, %0\n\t"
                 "s_nop 0\n\t"
                 "buffer_load_dword %1, %2, 0 offen lds"
                 :: "s"(lds_byte_addr), "v"(voff), "s"(rsrc) : "memory");
}

// The lean body (see spmm_tile) with the staging done by loads that write LDS
// directly.  A chunk stages 76 rows (19 16-byte pieces) of each of the 64
// columns, column after column without gaps: piece p = 19 * column + quad
// lives at byte 16 * p of the stage buffer, so load instruction i (lane l
// fetching piece 64 * i + l) fills bytes [1024 * i, 1024 * i + 1024) and 19
// instructions, every lane busy, stage the chunk.  Columns are then 76 floats
// apart, which keeps the 16-byte window reads (one lane per column) free of
// bank conflicts.  Wave w issues instructions w, w + 8 and (waves 0-2)
// w + 16; waves 3 and 4 (3 to 6 for tables with chunks longer than 8) fetch
// the chunk's diagonals for the 64 rows, 4 diagonals per instruction: 21 (23)
// loads per chunk, none through registers, no LDS write instruction.  Three LDS buffers: chunk k lives in buffer k % 3.
// The FMAs of chunk c are cut in two; between the halves sit the wait for
// chunk c+1, the barrier, the read of window(c+1) and the request for chunk
// c+3, while chunk c+2 is landing.
constexpr int SP_DQUADS = 19;                       // pieces per column staged by the direct loads (76 rows)
constexpr int SP_DPITCH = 4 * SP_DQUADS;            // floats between staged columns
constexpr int SP_DAVALS = SP_COLS * SP_DPITCH;      // diagonal values sit behind the dense rows
constexpr int SP_DSTAGE_FLOATS = SP_DAVALS + SP_AVALS;
static_assert(SP_COLS * SP_DQUADS % 64 == 0 && SP_ROWS + SP_CHUNK_MAX - 1 <= SP_DPITCH && SP_CHUNK_MAX <= SP_ADIAGS,
              "staging layout");

// INNER: every chunk the loop requests or reads (all but the first chunk walked) lies wholly inside the operand;
// the loop then carries neither the tests that tell such chunks from the others nor the code for the others.
// FIRST_ANY: the first chunk walked may cross an end of the operand (it is requested and read before the loop).
// `first` is the table position (relative to `chunks`) of the chunk to walk first, the others following in table
// order: a tile with one crossing chunk takes that one first and runs the INNER loop.  All chunks inside:
// <INNER, !FIRST_ANY>; one crossing chunk: <INNER, FIRST_ANY>; anything else: <!INNER, FIRST_ANY>, first = 0.
template <int LCK, int NTAB, bool EP, bool MIXED, bool INNER, bool FIRST_ANY>
__device__ __forceinline__ void spmm_tile_lean(
    float (&lds)[3][SP_DSTAGE_FLOATS], int row0, int col0,
    const Chunk *__restrict__ chunks, int nchunks, const float *__restrict__ vals, int stride,
    int ashift, const float *__restrict__ X, long long ldx, float *__restrict__ Y, long long ldy,
    int n_out, int n_in, int batch, float alpha, float beta, unsigned a_bytes, int first, int slot_step,
    SpEpilogue ep)
{
    constexpr int T = 8, WAVES = 8, CPW = SP_COLS / WAVES;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    float acc[T];
#pragma unroll
    for (int t = 0; t < T; ++t) acc[t] = 0.f;
    const int cols_here = min(SP_COLS, batch - col0);
    const unsigned x_bytes = (unsigned)(((long long)(cols_here - 1) * ldx + n_in) * 4);
    const float *xbase = X + (long long)col0 * ldx;

    // The result leaves in 16-byte stores, a lane holding 4 consecutive rows of
    // 2 columns (column wave*8 + lane/16 and the one 4 further), except when
    // samples are drawn: the generator yields 4 columns of one row per call,
    // so then a lane keeps one row and 8 columns.  Where beta scales the old
    // destination values they are requested now, in the same arrangement, and
    // their trip from memory overlaps the whole product.
    const bool by_row = EP && ep.act == 2;
    const int ecol = wave * CPW + (lane >> 4), erow = 4 * (lane & 15);
    float ypre[CPW];
#pragma unroll
    for (int q = 0; q < CPW; ++q) ypre[q] = 0.f;
    if (beta != 0.f) {
        const __amdgpu_buffer_rsrc_t yr = make_rsrc(
            Y + (long long)col0 * ldy, (unsigned)(((long long)(cols_here - 1) * ldy + n_out) * 4));
        if (by_row) {
#pragma unroll
            for (int q = 0; q < CPW; ++q) {
                const int col = wave * CPW + q;
                ypre[q] = buffer_load_f32(yr, col < cols_here ? (unsigned)(col * ldy + row0 + lane) * 4u : OOB_OFFSET);
            }
        } else {
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                const int col = ecol + 4 * k;
                const float4 v = buffer_load_f32x4(yr, col < cols_here ? (unsigned)(col * ldy + row0 + erow) * 4u : OOB_OFFSET);
                ypre[4 * k + 0] = v.x; ypre[4 * k + 1] = v.y; ypre[4 * k + 2] = v.z; ypre[4 * k + 3] = v.w;
            }
        }
    }

    // this lane's pieces in the three load instructions the wave issues
    unsigned x_off[3];
    unsigned x_lds[3];                      // byte offset inside a stage buffer that the instruction fills
    int x_quad[3];                          // the piece's place in its column (only chunks at the operand's ends ask)
#pragma unroll
    for (int it = 0; it < 3; ++it) {
        const int i = wave + WAVES * it;
        const int piece = 64 * i + lane;
        const int col = piece / SP_DQUADS, quad = piece - col * SP_DQUADS;
        x_off[it] = (unsigned)min(col, cols_here - 1) * ((unsigned)ldx * 4u) + 16u * quad;
        x_lds[it] = 1024u * i;
        x_quad[it] = quad;
    }
    // SP_COLS * SP_DQUADS / 64 = 19 instructions stage the dense rows of a chunk:
    // waves 0-2 issue three of them, the others two.  Waves 3 and 4 fetch the
    // chunk's diagonals instead, four diagonals x 64 rows each in one
    // instruction (lane = 16 * diagonal + 16-byte piece).  A load instruction
    // occupies the memory pipeline equally long whether it moves 4 or 16 bytes
    // per lane, so the count per chunk -- 21 -- is what matters.
    const bool x3 = wave < SP_DQUADS - 2 * WAVES;
    constexpr int A_LOADS = LCK > 8 ? 4 : 2;               // instructions that fetch diagonals: waves 3 .. 3 + A_LOADS - 1
    const bool a_wave = (wave >= 3) & (wave < 3 + A_LOADS);
    const int a_j = 4 * (wave - 3) + (lane >> 4);          // the diagonal this lane fetches (those waves)
    // every wave keeps its own count of loads per chunk: 3 for waves 0 .. 2 + A_LOADS, 2 for the others
    const bool three = wave < 3 + A_LOADS;

    const unsigned lds0 = (unsigned)(unsigned long long)(__attribute__((address_space(3))) float *)&lds[0][0];
    constexpr unsigned BUF_BYTES = SP_DSTAGE_FLOATS * 4u;

    // A chunk's table entry travels through three (four: chunks longer than 8) 16-byte SCALAR loads into
    // scalar registers, one iteration before the chunk is requested: no vector
    // memory instruction, no LDS copy and no register table stand between the
    // kernel's start and its first requests, and the loop's entries arrive
    // under the wait that ends every iteration anyway.
    struct Entry {
        int s0, len, p0, p1, p2, p3, p4, p5, p6, p7, p8, p9, p10, p11, p12;     // shift, length, table positions
    };
    auto fetch = [&](int c) __attribute__((always_inline)) {
        typedef int sp_i4 __attribute__((ext_vector_type(4)));
        typedef const sp_i4 __attribute__((address_space(4))) *sc_i4_ptr;
        int at = c;
        if constexpr (FIRST_ANY) at = c == 0 ? first : (c <= first ? c - 1 : c);       // `first` moved to the front
        at = min(at, nchunks - 1);
        const sc_i4_ptr e = (sc_i4_ptr)(chunks + at);
        const sp_i4 e0 = e[0], e1 = e[1], e2 = e[2];
        if constexpr (LCK > 8) {
            const sp_i4 e3 = e[3];
            return Entry{e0.x, e0.y, e0.z, e0.w, e1.x, e1.y, e1.z, e1.w, e2.x, e2.y, e2.z, e2.w, e3.x, e3.y, e3.z};
        } else {
            return Entry{e0.x, e0.y, e0.z, e0.w, e1.x, e1.y, e1.z, e1.w, e2.x, e2.y, -1, -1, -1, -1, -1};
        }
    };
    // requests chunk c, whose entry is en, into the buffer at byte address `buf`: 3 or 2 loads
    // two_c: std::true_type where the caller knows that this wave issues two loads per chunk (neither a third
    // piece of the dense rows nor diagonals), so that its copy of the loop carries no test for either
    // inner_c: std::true_type where the caller knows the chunk to lie wholly inside the operand
    auto issue = [&](int c, unsigned buf, const Entry &en, auto two_c, auto inner_c) __attribute__((always_inline)) {
        constexpr bool TWO = decltype(two_c)::value;
        constexpr bool IN = decltype(inner_c)::value;
        const int s0 = en.s0;
        const int a0 = row0 + s0;
        // past the table, and for a chunk whose rows lie outside the operand,
        // nothing is fetched: an empty resource delivers zeros
        const bool inside = IN || ((a0 >= 0) & (a0 + 4 * SP_DQUADS <= n_in));
        const bool outside = !IN && ((a0 + 4 * SP_DQUADS <= 0) | (a0 >= n_in));
        const bool real = (c < nchunks) & !outside;
        const sp_int4 xq = raw_rsrc(xbase, real ? x_bytes : 0u);
        if (LCK > 8 || (inside | !real)) {       // (longer chunks never come here crossing an end: see the kernel)
            const unsigned soff = (real & inside) ? (unsigned)a0 * 4u : 0u;
            lds_load_b128(xq, buf + x_lds[0], x_off[0], soff);
            lds_load_b128(xq, buf + x_lds[1], x_off[1], soff);
            if (!TWO && x3) lds_load_b128(xq, buf + x_lds[2], x_off[2], soff);
        } else {
            // The chunk's rows cross an end of the operand.  The staged block then starts at the multiple of
            // 4 at or below a0 (so that, the operand's row count being a multiple of 4 too, every 16-byte
            // piece lies wholly inside or wholly outside), each lane checks its own piece, and the pieces
            // outside arrive as zeros.  The same number of loads as for any other chunk: the waits still count.
            // Its diagonal values take a way of their own: where a diagonal leaves the matrix its storage holds
            // padding, and a 16-byte piece that crosses the first or last byte of the value array is answered
            // with zeros as a whole.  So every wave fetches the values of its own 8 rows one by one (lane =
            // 8 * diagonal + row, one more load for every wave; 0 where the product's input row does not
            // exist) into the upper half of the buffer's block of diagonal values, which chunks of at most 8
            // leave free.  A wait that counts one load too few only waits a little longer.
            {
                const int j = lane >> 3;
                int p[8] = {en.p0, en.p1, en.p2, en.p3, en.p4, en.p5, en.p6, en.p7};
#pragma unroll
                for (int k = 0; k < 8; ++k) asm("" : "+s"(p[k]));
                int sl = p[0];
#pragma unroll
                for (int k = 1; k < 8; ++k) sl = j == k ? p[k] : sl;
                const int orow = row0 + wave * T + (lane & (T - 1));
                const int in = orow + s0 + j;
                const bool ok = (j < en.len) & (sl >= 0) & ((unsigned)in < (unsigned)n_in);
                const unsigned off = ((unsigned)sl * (unsigned)stride + (unsigned)(ashift ? in : orow)) * 4u;
                lds_load_b32(raw_rsrc(vals, a_bytes), buf + (unsigned)(SP_DAVALS + 8 * SP_ROWS + 64 * wave) * 4u,
                             ok ? off : OOB_OFFSET);
            }
            const int a0p = a0 & ~3;
#pragma unroll
            for (int it = 0; it < 3; ++it) {
                const int r = a0p + 4 * x_quad[it];
                const bool ok = (r >= 0) & (r + 4 <= n_in);
                const unsigned voff = ok ? x_off[it] + (unsigned)(a0p * 4) : OOB_OFFSET;
                if (it < 2 || (!TWO && x3)) lds_load_b128(xq, buf + x_lds[it], voff, 0u);
            }
        }
        if (!TWO && a_wave) {
            // table position of this lane's diagonal, a_j: picked from the 8 scalars (each passed through an
            // empty asm so that the chain of selects stays one, and the entry stays in registers)
            constexpr int NP = LCK > 8 ? SP_CHUNK_MAX : 8;
            int p[SP_CHUNK_MAX] = {en.p0, en.p1, en.p2, en.p3, en.p4, en.p5, en.p6, en.p7, en.p8, en.p9, en.p10, en.p11, en.p12};
#pragma unroll
            for (int k = 0; k < NP; ++k) asm("" : "+s"(p[k]));
            int sl;
            if (slot_step != 0) {
                // the table's diagonals sit at evenly spaced positions inside every chunk: no picking
                sl = p[0] + a_j * slot_step;
            } else if constexpr (LCK <= 8) {
                // two waves fetch diagonals, four each: the wave's four candidates are chosen with scalar
                // selects (wave is uniform), the lane's own among them with three vector selects
                const bool up = wave != 3;
                int q[4] = {up ? p[4] : p[0], up ? p[5] : p[1], up ? p[6] : p[2], up ? p[7] : p[3]};
#pragma unroll
                for (int k = 0; k < 4; ++k) asm("" : "+s"(q[k]));
                const int jl = lane >> 4;
                sl = q[0];
#pragma unroll
                for (int k = 1; k < 4; ++k) sl = jl == k ? q[k] : sl;
            } else {
                sl = p[0];
#pragma unroll
                for (int k = 1; k < NP; ++k) sl = a_j == k ? p[k] : sl;
            }
            const bool ok = real & (a_j < en.len) & (sl >= 0);
            const int arow = row0 + erow + (ashift ? s0 + a_j : 0);          // first of the lane's 4 rows of its diagonal
            const unsigned voff = ok ? ((unsigned)sl * (unsigned)stride + (unsigned)arow) * 4u : OOB_OFFSET;
            lds_load_b128(raw_rsrc(vals, a_bytes), buf + (unsigned)(SP_DAVALS + 4 * (wave - 3) * SP_ROWS) * 4u, voff, 0u);
        }
    };
    // Reads the window of the chunk whose shift is s0.  A chunk that crosses an end of the operand was staged
    // from the multiple of 4 below its first row: its window starts up to 3 rows into the column (4-byte
    // reads then), and its diagonal values sit in the wave's own corner of the buffer (see issue).
    auto read_window = [&](SpWindow<LCK, T> &win, int b, int s0, auto inner_c) __attribute__((always_inline)) {
        constexpr bool IN = decltype(inner_c)::value;
        const float *buf = lds[b];
        const int a0 = row0 + s0;
        const bool inside = IN || ((a0 >= 0) & (a0 + 4 * SP_DQUADS <= n_in));
        const bool outside = !IN && ((a0 + 4 * SP_DQUADS <= 0) | (a0 >= n_in));
        if (LCK > 8 || (inside | outside)) {
            spmm_read_window<LCK, T>(win, buf + lane * SP_DPITCH + wave * T, buf + SP_DAVALS + wave * T + (lane & (T - 1)));
        } else {
            const float *src = buf + lane * SP_DPITCH + wave * T + (a0 & 3);
#pragma unroll
            for (int i = 0; i < T + LCK - 1; ++i) win.w[i] = src[i];
            const float *own = buf + SP_DAVALS + 8 * SP_ROWS + 64 * wave + (lane & (T - 1));
#pragma unroll
            for (int j = 0; j < LCK; ++j) win.a[j] = own[8 * j];
            // keeps this rare path apart from the one above: merged into one, both would read 4 bytes at a time
            asm volatile("");
        }
    };

    SpWindow<LCK, T> w0, w1;
    int s_cur, s_n1, s_n2;                  // shifts of the chunk whose window is read next, and of the two after it
    int l_cur, l_n1, l_n2;                  // lengths of the chunk whose FMAs run next, and of the two after it
    {
        const Entry h0 = fetch(0), h1 = fetch(1), h2 = fetch(2);
        issue(0, lds0, h0, std::false_type{}, std::integral_constant<bool, !FIRST_ANY>{});
        issue(1, lds0 + BUF_BYTES, h1, std::false_type{}, std::integral_constant<bool, INNER>{});
        issue(2, lds0 + 2 * BUF_BYTES, h2, std::false_type{}, std::integral_constant<bool, INNER>{});
        s_cur = h0.s0;
        s_n1 = h1.s0;
        s_n2 = h2.s0;
        l_cur = h0.len;
        l_n1 = h1.len;
        l_n2 = h2.len;
    }
    Entry e0 = fetch(3), e1 = e0;
    // The first window can be read as soon as chunk 0 (and the destination values) is in: the loads of
    // chunks 1 and 2 stay outstanding.
    if (three) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    __syncthreads();
    read_window(w0, 0, s_cur, std::integral_constant<bool, !FIRST_ANY>{});
    // Iteration c: buffers b (chunk c), b1 (chunk c+1); `use` is the entry of chunk c+3, `next` receives
    // the entry of chunk c+4.  The FMAs of chunk c are cut in two: the wait for chunk c+1, the barrier
    // and the read of its window sit between the halves, so the second half hides the read and a chunk
    // is waited for only when its turn has come -- the product starts with one chunk in LDS, not two.
    // The loop exists twice, for the waves that issue three loads per chunk and for those that issue two: the
    // waits are then fixed instructions, not a choice made in every iteration.
    constexpr int JH = (LCK + 1) / 2;
    auto run_loop = [&](auto three_c) __attribute__((always_inline)) {
    constexpr bool THREE = decltype(three_c)::value;
    auto iteration = [&](int c, int b, int b1, SpWindow<LCK, T> &cur, SpWindow<LCK, T> &nxt, const Entry &use, Entry &next) __attribute__((always_inline)) {
        spmm_rows_chunk<LCK, T, 0, JH, MIXED>(acc, cur, l_cur);
        // chunk c+1 must be in; the loads of chunk c+2 (requested whenever c+2 < 3 or it exists) may stay out
        const bool younger = (c + 2 < 3) | (c + 2 < nchunks);
        if (!younger) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        else if (THREE) asm volatile("s_waitcnt vmcnt(3) lgkmcnt(0)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(2) lgkmcnt(0)" ::: "memory");
        __syncthreads();                                 // also: every wave holds window(c), buffer b may be reused
        if (c + 1 < nchunks) read_window(nxt, b1, s_n1, std::integral_constant<bool, INNER>{});
        if (c + 3 < nchunks) issue(c + 3, lds0 + (unsigned)b * BUF_BYTES, use, std::integral_constant<bool, !THREE>{},
                                   std::integral_constant<bool, INNER>{});
        s_n1 = s_n2;
        s_n2 = use.s0;
        next = fetch(c + 4);
        spmm_rows_chunk<LCK, T, JH, LCK, MIXED>(acc, cur, l_cur);
        l_cur = l_n1;
        l_n1 = l_n2;
        l_n2 = use.len;
    };
    int c = 0, b = 0, b1 = 1, b2 = 2;
    if (nchunks & 1) {
        iteration(0, b, b1, w0, w1, e0, e1);
        { const SpWindow<LCK, T> t = w0; w0 = w1; w1 = t; }
        { const int t = b; b = b1; b1 = b2; b2 = t; }
        e0 = e1;
        c = 1;
    }
    for (; c < nchunks; c += 2) {
        iteration(c, b, b1, w0, w1, e0, e1);
        iteration(c + 1, b1, b2, w1, w0, e1, e0);
        { const int t0 = b, t1 = b1; b = b2; b1 = t0; b2 = t1; }
    }
    };
    if (three) run_loop(std::true_type{});
    else run_loop(std::false_type{});
    // every wave must be through with its window reads, and no load in flight, before the buffers are reused
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    float *out = &lds[0][0];
#pragma unroll
    for (int t = 0; t < T; ++t) out[lane * SP_OPITCH + wave * T + t] = acc[t];
    __syncthreads();
    if (by_row) {
        const long long row = (long long)row0 + lane;
        const float bias = ep.bias ? ep.bias[row] : 0.f;
        float v[CPW];
#pragma unroll
        for (int q = 0; q < CPW; ++q) v[q] = out[(wave * CPW + q) * SP_OPITCH + lane];   // all reads before the first store
        // the lane's 8 columns are two aligned blocks of 4: two generator calls
        SpRand4 rnd[CPW / 4];
#pragma unroll
        for (int k = 0; k < CPW / 4; ++k)
            rnd[k] = sp_philox((unsigned)row, (unsigned)(col0 + wave * CPW) / 4u + k, ep.seed_lo, ep.seed_hi);
#pragma unroll
        for (int q = 0; q < CPW; ++q) {
            const int col = wave * CPW + q;
            if (col0 + col < batch) {
                float *y = Y + (long long)(col0 + col) * ldy + row;
                const float r = (beta == 0.f) ? alpha * v[q] : beta * ypre[q] + alpha * v[q];
                stream_store(y, sp_finish(r, bias, ep.act, rnd[q / 4].w[q & 3]));
            }
        }
    } else {
        float4 bias4 = make_float4(0.f, 0.f, 0.f, 0.f);
        if (EP && ep.bias) {
            const float *bp = ep.bias + row0 + erow;
            bias4 = make_float4(bp[0], bp[1], bp[2], bp[3]);
        }
        float4 v[2];
#pragma unroll
        for (int k = 0; k < 2; ++k) v[k] = *reinterpret_cast<const float4 *>(out + (ecol + 4 * k) * SP_OPITCH + erow);
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const int col = ecol + 4 * k;
            if (col0 + col < batch) {
                const float s[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
                const float b4[4] = {bias4.x, bias4.y, bias4.z, bias4.w};
                float r[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float t = (beta == 0.f) ? alpha * s[e] : beta * ypre[4 * k + e] + alpha * s[e];
                    r[e] = EP ? sp_finish(t, b4[e], ep.act) : t;
                }
                stream_store4(Y + (long long)(col0 + col) * ldy + row0 + erow, r[0], r[1], r[2], r[3]);
            }
        }
    }
}

// EP = false: the plain product (no bias, no activation); EP = true applies `ep`.
// MIXED = true: the table has chunks shorter than LCK (their missing diagonals are skipped, see spmm_rows_chunk).
template <int LCK, int T, int NTAB, bool EP, bool MIXED>
__global__ __launch_bounds__(64 * SpShape<T>::WAVES, 4) void spmm_tiled_kernel(
    const Chunk *__restrict__ chunks, int nchunks, const float *__restrict__ vals, int stride,
    int ashift, const float *__restrict__ X, long long ldx, float *__restrict__ Y, long long ldy,
    int n_out, int n_in, int batch, float alpha, float beta, int col_tiles, int col_group, unsigned a_bytes,
    int s_min, int s_max, int period_tiles, int slot_step, SpEpilogue ep)
{
    static_assert(3 * SP_DSTAGE_FLOATS >= 2 * SP_STAGE_FLOATS, "the two bodies share one LDS block");
    __shared__ __attribute__((aligned(16))) float lds3[3][SP_DSTAGE_FLOATS];
    float (&lds)[2][SP_STAGE_FLOATS] = *reinterpret_cast<float (*)[2][SP_STAGE_FLOATS]>(&lds3[0][0]);
    const int tile = xcd_tile(blockIdx.x, gridDim.x);
    // Tiles are numbered column group by column group; inside a group of col_group column tiles the
    // column tile runs fastest, then the row tile.  The 64 tiles an XCD holds at a time are then
    // 64 / col_group neighbouring row tiles -- which share the dense rows of their bands -- of the same few
    // column tiles, however wide the batch is.
    int rowtile, coltile;
    if (col_group >= col_tiles) {
        rowtile = tile / col_tiles;
        coltile = tile - rowtile * col_tiles;
    } else {
        const int per_group = (int)(gridDim.x / (unsigned)col_tiles) * col_group;
        const int g = tile / per_group, in = tile - g * per_group;
        const int width = min(col_group, col_tiles - g * col_group);
        rowtile = in / width;
        coltile = g * col_group + (in - rowtile * width);
    }
    // A window table (window rows period_tiles tiles apart, period_tiles > 1): the tile one period down reads,
    // for window row dy, the dense rows this tile reads for dy + 1.  Inside every block of 16 periods the row
    // tiles are renumbered period-major -- position 16 r + m holds tile m * period_tiles + r -- so that the row
    // tiles an XCD holds at a time are 16 periods of one residue instead of 16 neighbours: tiles that run side
    // by side then ask for the block a neighbour in the walk fetched a chunk earlier, and find it in the L2.
    if (period_tiles > 1) {
        const int blk_tiles = 16 * period_tiles;
        const int blk = rowtile / blk_tiles, i = rowtile - blk * blk_tiles;
        const int row_tiles = (int)(gridDim.x / (unsigned)col_tiles);
        if ((blk + 1) * blk_tiles <= row_tiles) rowtile = blk * blk_tiles + (i & 15) * period_tiles + (i >> 4);
    }
    const int row0 = rowtile * SP_ROWS;
    const int col0 = coltile * SP_COLS;
    // The lean body serves a tile all of whose 64 output rows exist and none of
    // whose chunks straddles an end of the operand: each chunk's staged rows
    // [row0 + s0, row0 + s0 + 80) lie either inside it or wholly outside (such
    // a chunk contributes nothing and is skipped through an empty resource).
    bool lean = row0 + SP_ROWS <= n_out;
    int c_lo = 0, c_hi = nchunks;                   // the chunks with rows inside the operand: a contiguous
                                                    // range, the table being sorted by shift
    constexpr int STAGED = 4 * SP_DQUADS;           // rows the lean body stages per chunk
    // A chunk whose staged rows cross an end of the operand is staged from the multiple of 4 below its first
    // row, which costs up to 3 of the STAGED rows, and only works when no 16-byte piece crosses the end.
    // The lean body takes such chunks when they have at most 8 diagonals (their values are fetched into
    // the half of the buffer's diagonal block that longer chunks would need).
    const bool crossing_ok = (LCK <= 8) & ((n_in & 3) == 0);
    int crossing = 0, cross_at = nchunks;           // chunks crossing an end of the operand, and the first of them
    bool inner = true;                              // every walked chunk lies wholly inside the operand
    if (!((row0 + s_min >= 0) & (row0 + s_max + STAGED <= n_in))) {
        const int lane = threadIdx.x & 63;
        c_lo = nchunks;
        c_hi = 0;
#pragma unroll
        for (int k = 0; k < NTAB; ++k) {
            const int idx = 64 * k + lane;
            const int a0 = row0 + chunks[min(idx, nchunks - 1)].s0;
            const bool inside = (a0 >= 0) & (a0 + STAGED <= n_in);
            const bool outside = (a0 + STAGED <= 0) | (a0 >= n_in);
            const unsigned long long cm = __builtin_amdgcn_ballot_w64(!(inside | outside) & (idx < nchunks));
            crossing += (int)__builtin_popcountll(cm);
            if (cm) cross_at = min(cross_at, 64 * k + (int)__builtin_ctzll(cm));
            const unsigned long long m = __builtin_amdgcn_ballot_w64(!outside & (idx < nchunks));
            if (m) {
                c_lo = min(c_lo, 64 * k + (int)__builtin_ctzll(m));
                c_hi = max(c_hi, 64 * k + 64 - (int)__builtin_clzll(m));
            }
        }
        if (c_hi <= c_lo) {                          // nothing inside: one (outside) chunk keeps the pipeline fed
            c_lo = 0;
            c_hi = 1;
            inner = false;
        }
        inner &= crossing == 0;
        lean &= crossing == 0 || crossing_ok;
    }
    // only the chunks inside the operand are walked; the others would add zeros
    // A tile with one crossing chunk walks that chunk first: everything the loop then touches lies inside.
    if (lean && inner)
        spmm_tile_lean<LCK, NTAB, EP, MIXED, true, false>(lds3, row0, col0, chunks + c_lo, c_hi - c_lo, vals, stride, ashift, X,
                                                   ldx, Y, ldy, n_out, n_in, batch, alpha, beta, a_bytes, 0, slot_step, ep);
    else if (lean && crossing == 1 && c_hi > c_lo)
        spmm_tile_lean<LCK, NTAB, EP, MIXED, true, true>(lds3, row0, col0, chunks + c_lo, c_hi - c_lo, vals, stride, ashift, X,
                                                  ldx, Y, ldy, n_out, n_in, batch, alpha, beta, a_bytes,
                                                  cross_at - c_lo, slot_step, ep);
    else if (lean)
        spmm_tile_lean<LCK, NTAB, EP, MIXED, false, true>(lds3, row0, col0, chunks + c_lo, c_hi - c_lo, vals, stride, ashift, X,
                                                   ldx, Y, ldy, n_out, n_in, batch, alpha, beta, a_bytes, 0, slot_step, ep);
    else
        spmm_tile_edge<LCK, T, NTAB, EP, MIXED>(lds, row0, col0, chunks, nchunks, vals, stride, ashift, X, ldx, Y, ldy,
                                         n_out, n_in, batch, alpha, beta, a_bytes, ep);
}

#if CUVDIA_IN_PART(5)
// ------------------------------------------------------------ walking spmm --
//
// The product for *window* tables (plan_walk): k window rows `period` rows apart (repeated for every
// group).  Output tile m of a walk -- the tiles row_first + m * period, m = 0 .. S-1, of one column tile --
// reads, for window row dy of group g, the dense rows starting at
//     row_first + s0 + group_rows[g] + (m + dy) * period,
// so all the (m, dy) with m + dy = u read the SAME rows: block (u, g).  A workgroup walks u = 0 .. S+k-2
// and, for every group, stages block (u, g) ONCE -- its dense rows and the diagonal values of the up to k
// tiles that use it -- and applies it to those tiles, which it keeps alive as k sets of running sums
// (tile m in set m mod k).  One staged block, one window read and one barrier then serve up to k chunks
// instead of one: the staging per FMA drops k-fold against spmm_tile_lean, and what is left is the FMAs.
// A tile is complete when its window row k-1 has been applied (step u = m + k - 1): it is stored -- transposed
// through LDS, so that a lane writes 4 consecutive rows and a column's rows leave as one piece -- and its set
// starts the tile k steps on.  The walk is unrolled k steps deep so that every set has a static name.
//
// Workgroup = 8 waves x T rows (a tile of ROWS = 8 T output rows) x 64 batch columns, lanes <-> columns,
// diagonal values broadcast by DPP as in spmm_tile_lean.  Two LDS buffers: while block i is applied, block
// i+1 lands; one wait for everything in flight and one barrier per block.  Every block is staged from the
// multiple of 4 at or below its first row (a0 - SH; SH = a0 mod 4 is the same for every block of a product
// and a template parameter, so the window keeps static register indices): with a row count that is a
// multiple of 4 every 16-byte piece lies wholly inside the operand or outside, and the pieces outside arrive
// as zeros.  A block wholly outside the operand is skipped.  In a block that crosses an end of the operand
// the diagonal values of rows whose input row does not exist are padding: such a block's values are fetched
// element by element with that test (4-byte loads), every other block's as 16-byte pieces.
//
// Accumulation order per output element: window rows ascending, groups in table order within a window row
// (for tile m: blocks (m, 0), (m, 1), .., (m+1, 0), ..), diagonals ascending within a chunk -- the order of
// ascending shifts when there is one group, as in spmm_tile_lean.
template <int LCK, int K, int T, int SH>
struct WalkShape {
    static constexpr int WAVES = 8;                                         // waves per workgroup
    static constexpr int ROWS = WAVES * T;                                     // output rows per tile
    static constexpr int XNEED = SH + ROWS + LCK - 1;                       // staged dense rows that are read
    static constexpr int XQ = ((XNEED + 3) / 4) | 1;                        // 16-byte pieces per column, odd
    static constexpr int XPITCH = 4 * XQ;                                   // floats between staged columns
    static constexpr int XFLOATS = SP_COLS * XPITCH;
    static constexpr int DPI = 256 / ROWS;                                  // diagonals per 16-byte-piece instruction
    static constexpr int AI = (LCK + DPI - 1) / DPI;                        // such instructions per (tile, chunk)
    static constexpr int ATILE = AI * 256;                                  // floats per (tile, chunk) in LDS
    static constexpr int AFLOATS = K * ATILE;
    static constexpr int BUF_FLOATS = XFLOATS + AFLOATS;
    static constexpr int WIN = SH + T + LCK - 1;                            // window values a lane reads
    static constexpr int WQ = (WIN + 3) / 4;                                // as 16-byte reads
    static_assert(T == 8, "rows per wave");
    static constexpr int WGS_PER_CU = (160 * 1024) / (2 * BUF_FLOATS * 4) < 4 ? (160 * 1024) / (2 * BUF_FLOATS * 4) : 4;
    static_assert(ROWS - T + 4 * WQ <= XPITCH, "the last wave's window lies inside the staged column");
    static_assert(2 * BUF_FLOATS * 4 <= 80 * 1024, "two workgroups share a CU's LDS");
    static constexpr int WAVES_PER_SIMD = WGS_PER_CU * WAVES / 4 < 4 ? WGS_PER_CU * WAVES / 4 : 4;
};

// x / d == (x * m) >> 16 for every 0 <= x < limit
constexpr bool recip16_exact(unsigned d, unsigned m, unsigned limit)
{
    for (unsigned x = 0; x < limit; ++x)
        if (x / d != ((x * m) >> 16)) return false;
    return true;
}

// calls f(I) for I = 0 .. K-1 as compile-time constants
template <int K, int I, class F>
__device__ __forceinline__ void walk_for(F &&f)
{
    if constexpr (I < K) {
        f(std::integral_constant<int, I>{});
        walk_for<K, I + 1>(f);
    }
}
// calls step(u0 + UU, UU) for UU = 0 .. K-1 while u0 + UU < nsteps: the step's position in its group of K
// is a compile-time constant
template <int K, int UU, class F>
__device__ __forceinline__ void walk_steps(F &step, int u0, int nsteps)
{
    if constexpr (UU < K) {
        if (u0 + UU < nsteps) step(u0 + UU, std::integral_constant<int, UU>{});
        walk_steps<K, UU + 1>(step, u0, nsteps);
    }
}

// EP = true: a tile leaves through `ep` (a bias per output row and/or the logistic sigmoid).  A sampled result,
// ep.act == 2, leaves row by row instead -- a lane holds one row of its wave's 8 columns, two aligned blocks of 4,
// as the generator's counter (row, column / 4) wants them; 64 consecutive rows of a column per store.
template <int LCK, int K, int T, int SH, bool EP>
__global__ __launch_bounds__(512, (WalkShape<LCK, K, T, SH>::WAVES_PER_SIMD)) void spmm_walk_kernel(
    const int *__restrict__ tab,            // group_rows[ngroups], then aoff4[ngroups * K]
    int ngroups, int period, int s0, int astep4, int seg_tiles, const float *__restrict__ vals,
    const float *__restrict__ X, long long ldx, float *__restrict__ Y, long long ldy,
    int n_out, int n_in, int batch, float alpha, float beta, int col_tiles, unsigned a_bytes, SpEpilogue ep)
{
    typedef WalkShape<LCK, K, T, SH> S;
    constexpr int WAVES = S::WAVES, ROWS = S::ROWS, XQ = S::XQ, XPITCH = S::XPITCH, AI = S::AI, ATILE = S::ATILE, WQ = S::WQ;
    __shared__ __attribute__((aligned(16))) float lds[2][S::BUF_FLOATS];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

    // workgroup -> (segment, residue, column tile): the row tiles r, r + TP, r + 2 TP, .. (TP = period / ROWS) form
    // the walk of residue r; it is cut into segments of seg_tiles tiles
    const int tp = period / ROWS;
    const int wg = xcd_tile(blockIdx.x, gridDim.x);
    const int coltile = wg % col_tiles;
    const int rest = wg / col_tiles;
    const int res = rest % tp, seg = rest / tp;
    const int n_rt = n_out / ROWS;
    const int walk_len = (n_rt - res + tp - 1) / tp;              // tiles of this residue
    const int m0 = seg * seg_tiles;
    const int ntiles = min(seg_tiles, walk_len - m0);
    if (ntiles <= 0) return;
    const int row_first = (res + tp * m0) * ROWS;
    const int col0 = coltile * SP_COLS;
    const int cols_here = min(SP_COLS, batch - col0);
    const int nsteps = ntiles + K - 1;
    const int nblocks = nsteps * ngroups;

    // dense rows: instruction i = wave + WAVES it of a block stages pieces 64 i .. 64 i + 63, piece p = XQ * column + quad
    constexpr int XIT = (XQ + WAVES - 1) / WAVES;
    // A lane's share of the requests at the operand's ends is recomputed from its lane number for every block (a
    // few integer operations) rather than kept in registers across the walk: the running sums need them.
    auto lane_now = [&]() __attribute__((always_inline)) {
        int l = lane;
        asm volatile("" : "+v"(l));
        return l;
    };
    const unsigned x_bytes = (unsigned)(((long long)(cols_here - 1) * ldx + n_in) * 4);
    const sp_int4 xq = raw_rsrc(X + (long long)col0 * ldx, x_bytes);
    const sp_int4 aq = raw_rsrc(vals, a_bytes);
    const unsigned lds0 = (unsigned)(unsigned long long)(__attribute__((address_space(3))) float *)&lds[0][0];
    constexpr unsigned BUF_BYTES = S::BUF_FLOATS * 4u;

    typedef const int __attribute__((address_space(4))) *sc_int_ptr;
    const sc_int_ptr stab = (sc_int_ptr)tab;

    // piece -> column without an integer division: pieces number fewer than 2^11, and for those
    // piece / XQ == (piece * XQ_RECIP) >> 16 (checked below), a 24-bit multiplication at full rate
    constexpr unsigned XQ_RECIP = (65536u + XQ - 1) / XQ;
    static_assert(64 * XIT * WAVES <= 2048 && recip16_exact(XQ, XQ_RECIP, 2048), "piece / XQ by multiplication");
    // What a lane adds to the byte offset of a block that lies wholly inside the operand -- all but the few at
    // its ends -- is the same for the whole walk: its piece's column and place in the column for the dense rows,
    // its diagonal and rows for the values.  Kept in registers (5), a request of such a block costs one vector
    // addition instead of a dozen operations; the offsets stay vector offsets, so the buffer's range check
    // still answers anything out of range with zeros.
    constexpr int AIT = (K * S::AI + WAVES - 1) / WAVES;
    unsigned x_lane[XIT], a_lane[AIT];
#pragma unroll
    for (int it = 0; it < XIT; ++it) {
        const int piece = 64 * (wave + WAVES * it) + lane;
        const int col = (int)(__umul24((unsigned)piece, XQ_RECIP) >> 16);
        // (a column's last piece exists only to keep the pitch odd: where no window reaches it, it is not fetched)
        x_lane[it] = ((wave + WAVES * it < XQ) & (4 * (piece - col * XQ) < S::XNEED))
                         ? (unsigned)min(col, cols_here - 1) * ((unsigned)ldx * 4u) + 16u * (unsigned)(piece - col * XQ)
                         : OOB_OFFSET;
    }
#pragma unroll
    for (int k = 0; k < AIT; ++k) {
        const int n = wave + WAVES * k, h = n % S::AI;
        const int j = h * S::DPI + lane / (ROWS / 4);
        a_lane[k] = (n < K * S::AI && j < LCK) ? (unsigned)(16 * (lane % (ROWS / 4)) + j * astep4) : OOB_OFFSET;
    }
    // Requests block number i = u * ngroups + g (step u, group g) into buffer i & 1: its dense
    // rows and, for every tile m = u - dy that exists, the values of chunk (g, dy) for the tile's rows.
    auto issue = [&](int i, int u, int g) __attribute__((always_inline)) {
        const int a0 = row_first + s0 + stab[g] + u * period;        // first dense row the block's chunks read
        if (a0 + ROWS + LCK - 1 <= 0 || a0 >= n_in) return;          // wholly outside: nothing to stage (see apply)
        const unsigned buf = lds0 + (unsigned)(i & 1) * BUF_BYTES;
        const int a0p = a0 - SH;                                     // a multiple of 4
        if ((a0p >= 0) & (a0p + 4 * XQ <= n_in)) {
            // every staged piece exists
#pragma unroll
            for (int it = 0; it < XIT; ++it)
                if (wave + WAVES * it < XQ)
                    lds_load_b128(xq, buf + 1024u * (unsigned)(wave + WAVES * it), x_lane[it] + (unsigned)(a0p * 4), 0u);
        } else {
            const int ln = lane_now();
#pragma unroll
            for (int it = 0; it < XIT; ++it) {
                if (wave + WAVES * it < XQ) {
                    const int piece = 64 * (wave + WAVES * it) + ln;
                    const int col = (int)(__umul24((unsigned)piece, XQ_RECIP) >> 16);
                    const int r = a0p + 4 * (piece - col * XQ);
                    const unsigned x_col = (unsigned)min(col, cols_here - 1) * ((unsigned)ldx * 4u);
                    const bool ok = (r >= 0) & (r + 4 <= n_in) & (4 * (piece - col * XQ) < S::XNEED);
                    lds_load_b128(xq, buf + 1024u * (unsigned)(wave + WAVES * it), ok ? x_col + (unsigned)(r * 4) : OOB_OFFSET, 0u);
                }
            }
        }
        const bool inside = (a0 >= 0) & (a0 + ROWS + LCK - 1 <= n_in);
        const unsigned abuf = buf + (unsigned)S::XFLOATS * 4u;
        if (inside) {
            // 16-byte pieces: instruction n = dy * AI + h carries diagonals h*DPI .. of tile u - dy's chunk,
            // lane = (ROWS/4) * diagonal + piece
#pragma unroll
            for (int k = 0; k < AIT; ++k) {
                const int n = wave + WAVES * k;
                if (n >= K * AI) break;
                const int dy = n / AI;
                const int m = u - dy;
                if (m < 0 || m >= ntiles) continue;
                const unsigned base = (unsigned)(stab[ngroups + g * K + dy] + (row_first + m * period) * 4);   // wave-uniform
                lds_load_b128(aq, abuf + (unsigned)(n * 1024), a_lane[k] + base, 0u);
            }
        } else {
            const int ln = lane_now();
            // the block crosses an end of the operand: 4-byte loads, each lane testing its own element.
            // Instruction n = dy * NI + h carries EPI diagonals x ROWS rows, lane = ROWS * diagonal + row.
            constexpr int EPI = 64 / ROWS;                           // diagonals per instruction (1 or 2)
            constexpr int NI = (LCK + EPI - 1) / EPI;
            for (int n = wave; n < K * NI; n += WAVES) {
                const int dy = n / NI, h = n - dy * NI;
                const int m = u - dy;
                if (m < 0 || m >= ntiles) continue;
                const int j = h * EPI + ln / ROWS, i_row = ln % ROWS;
                const int in = a0 + i_row + j;                       // the input row this value multiplies
                const bool ok = (j < LCK) & ((unsigned)in < (unsigned)n_in);
                const int row = row_first + m * period + i_row;
                const unsigned off = (unsigned)(stab[ngroups + g * K + dy] + row * 4 + j * astep4);
                lds_load_b32(aq, abuf + (unsigned)((dy * ATILE + h * EPI * ROWS) * 4), ok ? off : OOB_OFFSET);
            }
        }
    };

    float acc[K][T];
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
        for (int t = 0; t < T; ++t) acc[k][t] = 0.f;

    // Applies block i = (u, g) to the tiles that use it; UU = u mod K gives the sets their static names:
    // tile m = u - dy sits in set (UU - dy) mod K.
    auto apply = [&](int i, int u, int g, auto uu_c) __attribute__((always_inline)) {
        constexpr int UU = decltype(uu_c)::value;
        const int a0 = row_first + s0 + stab[g] + u * period;
        if (a0 + ROWS + LCK - 1 <= 0 || a0 >= n_in) return;
        const float *buf = &lds[i & 1][0];
        float win[4 * WQ];
        {
            const float4 *p4 = reinterpret_cast<const float4 *>(buf + lane * XPITCH + wave * T);
#pragma unroll
            for (int q = 0; q < WQ; ++q) {
                const float4 v = p4[q];
                win[4 * q + 0] = v.x; win[4 * q + 1] = v.y; win[4 * q + 2] = v.z; win[4 * q + 3] = v.w;
            }
        }
        const float *abase = buf + S::XFLOATS + wave * T + (lane & (T - 1));
        auto fma_chunk = [&](float (&set)[T], const float (&a)[LCK]) __attribute__((always_inline)) {
            constexpr int NB = (LCK + 3) / 4;
            if constexpr (NB >= 1) fma_diagonals8<0, (LCK < 4 ? LCK : 4), SH>(set, a, win);
            if constexpr (NB >= 2) fma_diagonals8<4, (LCK < 8 ? LCK - 4 : 4), SH>(set, a, win);
            if constexpr (NB >= 3) fma_diagonals8<8, (LCK < 12 ? LCK - 8 : 4), SH>(set, a, win);
            if constexpr (NB >= 4) fma_diagonals8<12, LCK - 12, SH>(set, a, win);
        };
        // One path for every step: the values of chunk dy + 1 are read while chunk dy's FMAs run, whether or
        // not tile u - dy - 1 exists (the values of a tile that does not are whatever the buffer held, and are
        // not used); only the FMAs are skipped, so no running sum changes registers between the cases.
        float a[2][LCK];
#pragma unroll
        for (int j = 0; j < LCK; ++j) a[0][j] = abase[j * ROWS];
        walk_for<K, 0>([&](auto dy_c) __attribute__((always_inline)) {
            constexpr int dy = decltype(dy_c)::value;
            if constexpr (dy + 1 < K) {
#pragma unroll
                for (int j = 0; j < LCK; ++j) a[(dy + 1) & 1][j] = abase[(dy + 1) * ATILE + j * ROWS];
            }
            __builtin_amdgcn_sched_barrier(0);
            const int m = u - dy;
            if (m >= 0 && m < ntiles) fma_chunk(acc[((UU - dy) % K + K) % K], a[dy & 1]);
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    // The final store runs along the rows: 4 consecutive rows of a column per lane (LPC lanes per column, CPI
    // columns per instruction, NST instructions for the wave's CPW columns), after a transposition through LDS.
    constexpr int LPC = ROWS / 4, CPI = 64 / LPC, CPW = SP_COLS / WAVES, NST = CPW / CPI, OPITCH = ROWS + 4;
    static_assert(SP_COLS * OPITCH <= S::XFLOATS, "the transposition fits the dense rows' part of a buffer");
    typedef float f4u __attribute__((ext_vector_type(4), aligned(4)));
    typedef unsigned sp_u4 __attribute__((ext_vector_type(4)));
    // What a lane contributes to the addresses of a tile's final store, kept for the whole walk: where it writes
    // its sums in the transposition block and reads its 4 rows back (floats), and the byte offset of those rows in
    // the destination's column tile (the out-of-range marker for a column past the batch: the buffer store then
    // drops it).  A finished tile then costs its multiplications and two stores, no address arithmetic.
    const int o_write = lane * OPITCH + wave * T;
    int o_read[NST];
    unsigned y_lane[NST];
    {
        const int ecol = wave * CPW + lane / LPC, erow = 4 * (lane % LPC);
#pragma unroll
        for (int q = 0; q < NST; ++q) {
            const int col = ecol + CPI * q;
            o_read[q] = col * OPITCH + erow;
            y_lane[q] = col < cols_here ? (unsigned)(col * ldy + erow) * 4u : OOB_OFFSET;
        }
    }
    const __amdgpu_buffer_rsrc_t yr = make_rsrc(
        Y + (long long)col0 * ldy, (unsigned)(((long long)(cols_here - 1) * ldy + n_out) * 4));
    const bool by_row = EP && ep.act == 2;      // (kernel-uniform) the sampled result leaves row by row
    // Stores the tile that step u completes (m = u - K + 1, set (UU + 1) mod K) and clears its set for the tile
    // K steps on.  `ilast` is the step's last block: every wave is through with its buffer (the barrier that
    // ended the block), and the next request into it comes after the second barrier below.
    auto finish = [&](int u, int ilast, auto uu_c, const f4u (&ypre)[NST]) __attribute__((always_inline)) {
        constexpr int SET = (decltype(uu_c)::value + 1) % K;
        const int m = u - (K - 1);
        if (m >= 0 && m < ntiles) {
            float *out = &lds[ilast & 1][0];
            static_assert(OPITCH % 4 == 0 && T % 4 == 0, "the sums leave as 16-byte LDS writes");
#pragma unroll
            for (int t = 0; t < T; t += 4)
                *reinterpret_cast<float4 *>(out + o_write + t) =
                    make_float4(acc[SET][t], acc[SET][t + 1], acc[SET][t + 2], acc[SET][t + 3]);
            __syncthreads();
            if (EP && by_row) {
                static_assert(CPW == 4 * NST && CPW % 4 == 0 && ROWS == 64, "a row per lane, the wave's columns in blocks of 4");
                float vv[CPW];
#pragma unroll
                for (int q = 0; q < CPW; ++q) vv[q] = out[(wave * CPW + q) * OPITCH + lane];
                const unsigned row = (unsigned)(row_first + m * period + lane);
                const float bias = ep.bias ? ep.bias[row] : 0.f;
                SpRand4 rnd[CPW / 4];
#pragma unroll
                for (int k = 0; k < CPW / 4; ++k)
                    rnd[k] = sp_philox(row, (unsigned)(col0 + wave * CPW) / 4u + k, ep.seed_lo, ep.seed_hi);
                const float yp[CPW] = {ypre[0].x, ypre[0].y, ypre[0].z, ypre[0].w, ypre[1].x, ypre[1].y, ypre[1].z, ypre[1].w};
                const unsigned tile_off = (unsigned)(row_first + m * period) * 4u;  // wave-uniform
#pragma unroll
                for (int q = 0; q < CPW; ++q) {
                    const int col = wave * CPW + q;                                 // wave-uniform
                    if (col < cols_here) {
                        const float r = (beta == 0.f) ? alpha * vv[q] : beta * yp[q] + alpha * vv[q];
                        __builtin_amdgcn_raw_buffer_store_b32(
                            __builtin_bit_cast(unsigned, sp_finish(r, bias, ep.act, rnd[q / 4].w[q & 3])), yr,
                            (unsigned)lane * 4u, tile_off + (unsigned)(col * ldy) * 4u, 2);
                    }
                }
                __syncthreads();
#pragma unroll
                for (int t = 0; t < T; ++t) acc[SET][t] = 0.f;
                return;
            }
            f4u v[NST];
#pragma unroll
            for (int q = 0; q < NST; ++q) v[q] = *reinterpret_cast<const f4u *>(out + o_read[q]);
            const unsigned tile_off = (unsigned)(row_first + m * period) * 4u;      // wave-uniform
            if (beta == 0.f) {
#pragma unroll
                for (int q = 0; q < NST; ++q) v[q] = alpha * v[q];
            } else {
#pragma unroll
                for (int q = 0; q < NST; ++q) v[q] = beta * ypre[q] + alpha * v[q];
            }
            if constexpr (EP) {
                // the lane's 4 rows are the same in every column it stores: one bias value each
                float b4[4] = {0.f, 0.f, 0.f, 0.f};
                if (ep.bias) {
                    const float *bp = ep.bias + (row_first + m * period) + 4 * (lane % LPC);
#pragma unroll
                    for (int e = 0; e < 4; ++e) b4[e] = bp[e];
                }
#pragma unroll
                for (int q = 0; q < NST; ++q)
                    v[q] = f4u{sp_finish(v[q].x, b4[0], ep.act), sp_finish(v[q].y, b4[1], ep.act),
                               sp_finish(v[q].z, b4[2], ep.act), sp_finish(v[q].w, b4[3], ep.act)};
            }
#pragma unroll
            for (int q = 0; q < NST; ++q)       // non-temporal, like every result of the library
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(sp_u4, v[q]), yr, y_lane[q], tile_off, 2);
            __syncthreads();
        }
#pragma unroll
        for (int t = 0; t < T; ++t) acc[SET][t] = 0.f;
    };

    issue(0, 0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    auto step = [&](int u, auto uu_c) __attribute__((always_inline)) {
        // destination values of the tile this step completes (beta != 0), requested ahead of its last blocks
        f4u ypre[NST];
#pragma unroll
        for (int q = 0; q < NST; ++q) ypre[q] = f4u{0.f, 0.f, 0.f, 0.f};
        const int mf = u - (K - 1);
        if (beta != 0.f && mf >= 0 && mf < ntiles) {
            const unsigned tile_off = (unsigned)(row_first + mf * period) * 4u;
            if (EP && by_row) {
                // (the row-by-row exit: this lane's row of the wave's 8 columns)
                float yp[CPW];
#pragma unroll
                for (int q = 0; q < CPW; ++q) {
                    const int col = wave * CPW + q;
                    yp[q] = col < cols_here ? __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                  yr, (unsigned)lane * 4u, tile_off + (unsigned)(col * ldy) * 4u, 0))
                                            : 0.f;
                }
                ypre[0] = f4u{yp[0], yp[1], yp[2], yp[3]};
                ypre[1] = f4u{yp[4], yp[5], yp[6], yp[7]};
            } else {
#pragma unroll
                for (int q = 0; q < NST; ++q)
                    ypre[q] = __builtin_bit_cast(f4u, __builtin_amdgcn_raw_buffer_load_b128(yr, y_lane[q], tile_off, 0));
            }
        }
        int i = u * ngroups;
        for (int g = 0; g < ngroups; ++g, ++i) {
            if (i + 1 < nblocks) {
                const bool last = g + 1 == ngroups;
                issue(i + 1, last ? u + 1 : u, last ? 0 : g + 1);
            }
            apply(i, u, g, uu_c);
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __syncthreads();
        }
        finish(u, i - 1, uu_c, ypre);
    };
    for (int u0 = 0; u0 < nsteps; u0 += K) walk_steps<K, 0>(step, u0, nsteps);
}
#endif  // part 5

// ------------------------------------------------------------ tiled dd2dia --
//
// Workgroup = 256 rows of ONE unit: a run chunk, or two chunks whose first
// shifts differ by delta (a multiple of 4) -- e.g. two rows of a 2-d window
// (what follows describes pairs up to 128 rows apart; DdShape lists the other
// forms).  Lane l owns rows row0 + 4l .. 4l+3 and 4 x LC partial sums per
// chunk (LC = the longest chunk of the table; positions past a chunk's own
// length are computed and dropped).  A table with runs of more than 8 shifts
// (window rows wider than 8) is walked in the products' chunks of up to 13
// instead, every unit one such chunk: as many sums as a pair, one band, one
// copy of A's rows.  A single chunk is worked by 4 waves, a pair by 8; wave
// q walks the batch-column groups g = q, q + WAVES, ...
// (4 columns per group).  Per group and column the wave
//   1. writes the column's rows [row0 + s0, row0 + s0 + 264 + delta) of B,
//      fetched one step earlier as 16-byte pieces (a lane holds 4 consecutive
//      rows, two loads per column), to its private LDS buffer -- no workgroup
//      barrier in the loop.  Rows of that band outside B are not masked: they
//      only meet sums of slots that hold no matrix element (see the loads);
//   2. reads its 4 + LC - 1 wide window of B per chunk from LDS with 16-byte
//      reads (the second chunk's window starts delta rows further);
//   3. requests the same column of the next group: its rows of B and its own
//      4 rows of A (one 16-byte load when A allows it).  Columns past the
//      batch go through an empty buffer resource and come back as zeros
//      without touching memory, so the loop body never branches and every
//      wait counts exactly;
//   4. issues 4 x LC FMAs per chunk.  A pair needs A once and the two bands of
//      B overlap, so it moves about 40 % fewer bytes per FMA than two singles.
// At the end the waves' partial sums meet in LDS and are added in a fixed
// order; the result is written with lanes along rows (the values of C that
// beta scales were fetched at kernel start).

constexpr int DD_ROWS = 256;
constexpr int DD_BG = 4;           // batch columns per step

// LC > CHUNK_MAX: the unit is one long chunk of the products' table (up to
// SP_CHUNK_MAX shifts: a whole row of a wide 2-d window), never a pair.  It
// keeps as many running sums as a pair but is worked by 4 waves: three such
// workgroups share a CU (registers allow 3 waves per SIMD, and the block the
// sums are added in is kept just under a third of the CU's LDS).
// WIDE says how a pair is served.  The two chunks of a pair start delta rows apart; for row i the first pairs it
// with rows i + s0 + j of B, the second with rows i + s0 + delta + j.
//   DD_NARROW, DD_WIDE -- both chunks work on the SAME rows of A: one copy of A's rows and one band of B that
//     holds both windows, delta rows apart (two 16-byte pieces per lane and column up to PAIR_NARROW_DELTA, a
//     third up to PAIR_BAND_DELTA: window rows of a map wider than 128); 8 waves, alone on their CU;
//   DD_SHIFTED -- the second chunk works on the rows delta ABOVE the first's, so that both read the SAME rows of B:
//     one band of one piece (the tile is cut short, dd_short_rows), one window per column for both chunks, and two
//     copies of A's rows.  Any distance that is a multiple of 4; 4 waves, three such workgroups to a CU.
constexpr int DD_NARROW = 0, DD_WIDE = 1, DD_SHIFTED = 2;
template <int NCH, int LC, int WIDE = DD_NARROW>
struct DdShape {
    static_assert(NCH == 1 || LC <= CHUNK_MAX, "pairs are made of short chunks");
    static_assert(NCH == 2 || WIDE == DD_NARROW, "only pairs come in forms");
    static constexpr bool LONG = LC > CHUNK_MAX;
    static constexpr int SPAN = LONG ? SP_CHUNK_MAX : CHUNK_MAX;    // shifts a chunk can have
    static constexpr int NQ = (NCH == 1 || WIDE == DD_SHIFTED) ? 4 : WIDE == DD_WIDE ? 8 : 6;   // 64-row blocks of the band
    static constexpr int NB = WIDE == DD_WIDE ? 3 : WIDE == DD_SHIFTED ? 1 : 2;   // 16-byte pieces a lane holds per column
    static constexpr int PITCH = 64 * NQ + (LONG ? 16 : 8);     // staged rows per column: 264, 272, 392 or 520
    static constexpr int WAVES = (NCH == 2 && WIDE != DD_SHIFTED) ? 8 : 4;
    static constexpr int RED_PAD = LONG ? 4 : 8;              // a long chunk's sums then fit a third of a CU's LDS
    static constexpr int WAVE_FLOATS = 2 * DD_BG * PITCH + 4;   // two buffers + a slot idle lanes write to
    static constexpr int STAGE_FLOATS = WAVES * WAVE_FLOATS;
};
static_assert(DdShape<2, CHUNK_MAX>::PITCH >= DD_ROWS + PAIR_NARROW_DELTA + CHUNK_MAX, "a pair's band must fit its buffer");
static_assert(DdShape<2, CHUNK_MAX, DD_WIDE>::PITCH >= DD_ROWS + PAIR_BAND_DELTA + CHUNK_MAX, "a wide pair's band must fit its buffer");
static_assert(DdShape<2, CHUNK_MAX>::NB == 2 && DdShape<2, CHUNK_MAX, DD_WIDE>::NB == 3 && DdShape<1, CHUNK_MAX>::NB == 2, "pieces per lane");
static_assert(DdShape<1, SP_CHUNK_MAX>::PITCH >= DD_ROWS + 4 * ((4 + SP_CHUNK_MAX - 1 + 3) / 4) - 4,
              "a long chunk's last window must fit its buffer");

// What a wave has in flight of A for one group of 4 batch columns (two of
// these alternate; B's pieces need one set of registers only, see the loop).
template <int NA>
struct DdStage {
    float a[NA][DD_BG][4];    // this lane's 4 rows of each column (a shifted pair: and the 4 rows delta above)
};

template <int LC, int NCH>
constexpr int dd_red_floats() { return 4 * 4 * (NCH * LC * 64 + DdShape<NCH, LC>::RED_PAD); }
template <int LC, int NCH, int WIDE = DD_NARROW>
constexpr int dd_lds_floats()
{
    // (a shifted pair adds its chunks' sums one chunk after the other, in the block of a single chunk)
    constexpr int red = WIDE == DD_SHIFTED ? dd_red_floats<LC, 1>() : dd_red_floats<LC, NCH>();
    return DdShape<NCH, LC, WIDE>::STAGE_FLOATS > red ? DdShape<NCH, LC, WIDE>::STAGE_FLOATS : red;
}

// Rows of a tile.  A launch of single chunks only (no pairs) cuts its tiles 8 (long chunks: 16) rows short of
// 256: the band of B a tile needs -- its rows plus the chunk's span -- then fits the 256 rows that one 16-byte
// piece per lane covers, and a column costs two load instructions (B, A) instead of three.
template <int LC>
constexpr int dd_short_rows() { return DD_ROWS - (LC > CHUNK_MAX ? 16 : 8); }

template <int LC, int NCH, bool AVEC, int WIDE = DD_NARROW, bool SHORT = false>
__device__ __forceinline__ void dd2dia_unit(
    float *lds, int row0, const Chunk *ck1, const Chunk *ck2, float *__restrict__ C, int stride,
    const float *__restrict__ A, long long lda, const float *__restrict__ B, long long ldb,
    int h, int w, int batch, float alpha, float beta, unsigned a_bytes, unsigned b_bytes,
    unsigned c_bytes)
{
    typedef DdShape<NCH, LC, WIDE> S;
    constexpr bool SHIFTED = WIDE == DD_SHIFTED;
    static_assert(!SHORT || NCH == 1, "short tiles: launches of single chunks, and of shifted pairs (which say so)");
    static_assert(!SHIFTED || AVEC, "pairs are formed with 16-byte loads of A only");
    constexpr int TR = (SHORT || SHIFTED) ? dd_short_rows<LC>() : DD_ROWS;    // rows of the tile
    constexpr int PITCH = S::PITCH, WAVES = S::WAVES, NB = SHORT ? 1 : S::NB;
    constexpr int NA = SHIFTED ? 2 : 1;                      // copies of A's rows a lane holds per column
    constexpr int NWIN = SHIFTED ? 1 : NCH;                  // windows of B a lane reads per column
    constexpr int NRED = SHIFTED ? 1 : NCH;                  // chunks whose sums meet in LDS at a time
    static_assert(!SHORT || TR + S::SPAN <= 256 || (S::LONG && TR + 16 <= 256), "a short tile's band is one piece per lane");
    constexpr int WIN = 4 + LC - 1;
    constexpr int WQ = (WIN + 3) / 4;
    constexpr int RED_T = NRED * LC * 64 + S::RED_PAD;       // floats between the 4 rows a lane owns: keeps the
                                                    // row-major read below free of bank conflicts
    constexpr int RED_WAVE = 4 * RED_T;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // each table entry in three (a long chunk: four) 16-byte scalar loads
    typedef int int4v __attribute__((ext_vector_type(4)));
    typedef const int4v __attribute__((address_space(4))) *sc_int4_ptr;
    int s0[NCH], slots[NCH][S::SPAN];
#pragma unroll
    for (int n = 0; n < NCH; ++n) {
        const sc_int4_ptr e = (sc_int4_ptr)(n == 0 ? ck1 : ck2);
        const int4v e0 = e[0], e1 = e[1], e2 = e[2];
        s0[n] = e0.x;
        slots[n][0] = e0.z; slots[n][1] = e0.w; slots[n][2] = e1.x; slots[n][3] = e1.y;
        slots[n][4] = e1.z; slots[n][5] = e1.w; slots[n][6] = e2.x; slots[n][7] = e2.y;
        if constexpr (S::LONG) {
            const int4v e3 = e[3];
            slots[n][8] = e2.z; slots[n][9] = e2.w; slots[n][10] = e3.x; slots[n][11] = e3.y; slots[n][12] = e3.z;
        }
    }
    const int delta = NCH == 2 ? s0[NCH - 1] - s0[0] : 0;      // rows between the two windows
    const int wdelta = SHIFTED ? 0 : delta;                     // .. inside the staged band
    const int need = TR + wdelta + S::SPAN;                     // staged rows that are ever read
    const int base = row0 + s0[0];                              // first staged row of B
    // Every slot of the unit pairs row i with row i + s0 + j of B: with the
    // whole band outside B the unit stores no matrix element, and there is
    // nothing to compute or to write (the whole workgroup leaves together).
    if (base + need <= 0 || base >= w) return;
    // .. and with every row of the tile (a shifted pair: and every row delta above) past A's last
    if (row0 - (SHIFTED ? delta : 0) >= h) return;
    const int myrow = row0 + 4 * lane;

    // C values this lane will combine at the end: row row0 + 64*wave + lane of
    // every diagonal of the unit (waves 0..3; a pair's waves 4..7 leave the
    // output to them).  Byte offset of that slot, or the out-of-range marker
    // where no matrix element sits.
    auto c_offset = [&](int n, int j) -> unsigned {
        const int sl = slots[n][j];
        const int o = row0 + 64 * wave + lane - ((SHIFTED && n) ? delta : 0);
        const int in = o + s0[n] + j;
        const bool ok = (wave < 4) & (sl >= 0) & (o >= 0) & (o < h) & (in >= 0) & (in < w) & (64 * wave + lane < TR);
        return ok ? ((unsigned)sl * (unsigned)stride + (unsigned)o) * 4u : OOB_OFFSET;
    };
    float cpre[NCH][LC];
#pragma unroll
    for (int n = 0; n < NCH; ++n)
#pragma unroll
        for (int j = 0; j < LC; ++j) cpre[n][j] = 0.f;
    // beta == 0: C is not read; waves 4..7 of a pair write nothing and ask for nothing (a load costs the
    // memory pipeline its slot even when every lane is out of range)
    if ((beta != 0.f) & (wave < 4)) {
        const __amdgpu_buffer_rsrc_t cr = make_rsrc(C, c_bytes);
#pragma unroll
        for (int n = 0; n < NCH; ++n)
#pragma unroll
            for (int j = 0; j < LC; ++j) cpre[n][j] = buffer_load_f32(cr, c_offset(n, j));
    }

    // The band of B travels as 16-byte pieces, a lane holding rows base + 4*lane
    // .. + 3 and, where the band reaches that far, base + 256 + 4*lane .. + 3
    // (a wide pair: and base + 512 + 4*lane .. + 3):
    // two (three) loads per column, whatever the alignment of base (a load instruction
    // occupies the memory pipeline equally long for 4 and for 16 bytes per
    // lane).  Rows of the band outside B need no care in general: they only
    // meet sums of slots that hold no matrix element and are never stored, and
    // a piece that leaves column c lands in a neighbouring column of the same
    // allocation.  The whole byte offset goes into the vector operand, which
    // is what the buffer's range check looks at, so nothing outside the
    // allocation is ever touched.  Only where a column's band crosses the
    // allocation's first or last byte (the first and the last batch columns of
    // tiles at the ends of B) a piece could lose valid rows to the range check,
    // which answers for the piece as a whole: those columns -- [0, rare_lo) and
    // [rare_hi, batch) -- stay out of the pipelined loop and are worked row by
    // row by wave 0 before it (see below).
    const int nquad = (need + 3) / 4;                     // pieces per column that are ever read, 66 .. 130
    const bool tail = lane < nquad - 64;
    const bool tail2 = lane < nquad - 128;                // a wide pair's third piece
    const unsigned vb_off0 = (unsigned)(base + 4 * lane) * 4u;
    const long long b_floats = (long long)(batch - 1) * ldb + w;
    // column c's band starts c*ldb + base floats into the allocation and is 4*nquad floats long
    int rare_lo = 0, rare_hi = batch;
    if (base < 0) rare_lo = (int)min((long long)batch, (-(long long)base + ldb - 1) / ldb);
    {
        const long long room = b_floats - base - 4 * nquad;                   // c*ldb must not exceed this
        if (room < (long long)(batch - 1) * ldb) rare_hi = room < 0 ? 0 : (int)(room / ldb) + 1;
        rare_hi = max(rare_hi, rare_lo);
    }
    unsigned a_off[4];
    unsigned a_off2 = OOB_OFFSET;                     // a shifted pair: the rows delta above (delta is a multiple of 4)
    if (SHIFTED) a_off2 = ((myrow - delta >= 0) & (myrow - delta + 3 < h) & (4 * lane + 3 < TR)) ? (unsigned)(myrow - delta) * 4u : OOB_OFFSET;
    if (AVEC) {
        a_off[0] = ((myrow + 3 < h) & (4 * lane + 3 < TR)) ? (unsigned)myrow * 4u : OOB_OFFSET;
    } else {
#pragma unroll
        for (int t = 0; t < 4; ++t) a_off[t] = ((myrow + t < h) & (4 * lane + t < TR)) ? (unsigned)(myrow + t) * 4u : OOB_OFFSET;
    }
    // Column strides in bytes, pinned to scalar registers: they feed the loads'
    // scalar offsets, and left alone the compiler derives them from a vector
    // copy of ldb and then has to loop over lanes to issue each load.
    unsigned lda4, ldb4;
    asm("v_readfirstlane_b32 %0, %1" : "=s"(lda4) : "v"((unsigned)lda * 4u));
    asm("v_readfirstlane_b32 %0, %1" : "=s"(ldb4) : "v"((unsigned)ldb * 4u));

    float acc[NCH][4][LC];
#pragma unroll
    for (int n = 0; n < NCH; ++n)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int j = 0; j < LC; ++j) acc[n][t][j] = 0.f;

    const int ngroups = (batch + DD_BG - 1) / DD_BG;
    const int steps = (ngroups + WAVES - 1) / WAVES;        // same for every wave
    float *mybuf = lds + wave * S::WAVE_FLOATS;
    const __amdgpu_buffer_rsrc_t b_all = make_rsrc(B, b_bytes);

    // B in flight: per column, rows base + 4*lane .. + 3 and base + 256 + 4*lane .. + 3 of the band.  One set
    // serves the current and the next group: column i of the next group is requested after column i of the
    // current one has gone to LDS.
    float4 bq[DD_BG][NB];
    // requests column i of group g: B rows into bq, A rows into st.a
    const unsigned rare_span = (unsigned)(rare_hi - rare_lo);
    auto issue_col = [&](int g, int i, DdStage<NA> &st) {
        const int b0 = __builtin_amdgcn_readfirstlane(g * DD_BG);   // wave-uniform: keeps column offsets scalar
        const int col = b0 + i;
        const bool live = (unsigned)(col - rare_lo) < rare_span;      // rare_lo <= col < rare_hi in one compare
        const __amdgpu_buffer_rsrc_t br = make_rsrc(B, live ? b_bytes : 0u);
        const unsigned colb = (unsigned)col * ldb4;
        const unsigned v0 = vb_off0 + colb;
        bq[i][0] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(br, v0, 0, 0));
        if constexpr (NB >= 2)
            bq[i][1] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(br, tail ? v0 + 1024u : OOB_OFFSET, 0, 0));
        if constexpr (NB == 3)
            bq[i][2] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(br, tail2 ? v0 + 2048u : OOB_OFFSET, 0, 0));
        const __amdgpu_buffer_rsrc_t ar = make_rsrc(A, live ? a_bytes : 0u);
        const unsigned cola = (unsigned)col * lda4;
        if (AVEC) {
            const float4 v = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(ar, a_off[0], cola, 0));
            st.a[0][i][0] = v.x; st.a[0][i][1] = v.y; st.a[0][i][2] = v.z; st.a[0][i][3] = v.w;
            if constexpr (SHIFTED) {
                const float4 u = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(ar, a_off2, cola, 0));
                st.a[1][i][0] = u.x; st.a[1][i][1] = u.y; st.a[1][i][2] = u.z; st.a[1][i][3] = u.w;
            }
        } else {
#pragma unroll
            for (int t = 0; t < 4; ++t)
                st.a[0][i][t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ar, a_off[t], cola, 0));
        }
    };
    auto issue = [&](int g, DdStage<NA> &st) {
#pragma unroll
        for (int i = 0; i < DD_BG; ++i) issue_col(g, i, st);
    };
    auto commit_col = [&](int par, int i) {
        float *buf = mybuf + par * (DD_BG * PITCH);
        *reinterpret_cast<float4 *>(buf + i * PITCH + 4 * lane) = bq[i][0];
        // lanes past the band's end drop their (zero) piece in the spare slot
        if constexpr (NB >= 2)
            *reinterpret_cast<float4 *>(tail ? buf + i * PITCH + 256 + 4 * lane : mybuf + 2 * DD_BG * PITCH) = bq[i][1];
        if constexpr (NB == 3)
            *reinterpret_cast<float4 *>(tail2 ? buf + i * PITCH + 512 + 4 * lane : mybuf + 2 * DD_BG * PITCH) = bq[i][2];
        wave_lds_fence();
    };
    struct Windows { float w[NWIN][WQ * 4]; };
    auto read_windows = [&](Windows &win, const float *buf, int i) {
#pragma unroll
        for (int n = 0; n < NWIN; ++n) {
            const float4 *p4 = reinterpret_cast<const float4 *>(buf + i * PITCH + 4 * lane + (n ? delta : 0));
#pragma unroll
            for (int q = 0; q < WQ; ++q) {
                const float4 v = p4[q];
                win.w[n][4 * q + 0] = v.x; win.w[n][4 * q + 1] = v.y; win.w[n][4 * q + 2] = v.z; win.w[n][4 * q + 3] = v.w;
            }
        }
    };
    // column i of a stage: the first chunk on the lane's rows; the second on the same rows and its own window,
    // or (a shifted pair) on the rows delta above and the same window
    auto fmas = [&](const DdStage<NA> &st, int i, const Windows &win) {
#pragma unroll
        for (int n = 0; n < NCH; ++n)
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int j = 0; j < LC; ++j)
                    acc[n][t][j] = __builtin_fmaf(st.a[SHIFTED ? n : 0][i][t], win.w[SHIFTED ? 0 : n][t + j], acc[n][t][j]);
    };
    // Step k works on group wave + WAVES*k out of stage set k & 1 and LDS
    // buffer k & 1, one column at a time: column i's rows of B go to LDS and
    // its windows are read back while the FMAs of column i - 1 run; column i
    // of the next group is requested right after, so every load has one whole
    // step to arrive and the requests are spread between the FMA blocks.  Past
    // the last group the requests hit the empty resource.
    auto step = [&](int k, int par, DdStage<NA> &cur, DdStage<NA> &nxt) {
        const float *buf = mybuf + par * (DD_BG * PITCH);
        const int gn = wave + WAVES * (k + 1);
        Windows w0, w1;
        commit_col(par, 0);
        read_windows(w0, buf, 0);
        commit_col(par, 1);
        read_windows(w1, buf, 1);
        issue_col(gn, 0, nxt);
        __builtin_amdgcn_sched_barrier(0);
        fmas(cur, 0, w0);
        __builtin_amdgcn_sched_barrier(0);
        commit_col(par, 2);
        read_windows(w0, buf, 2);
        issue_col(gn, 1, nxt);
        __builtin_amdgcn_sched_barrier(0);
        fmas(cur, 1, w1);
        __builtin_amdgcn_sched_barrier(0);
        commit_col(par, 3);
        read_windows(w1, buf, 3);
        issue_col(gn, 2, nxt);
        __builtin_amdgcn_sched_barrier(0);
        fmas(cur, 2, w0);
        __builtin_amdgcn_sched_barrier(0);
        issue_col(gn, 3, nxt);
        __builtin_amdgcn_sched_barrier(0);
        fmas(cur, 3, w1);
        __builtin_amdgcn_sched_barrier(0);
    };

    DdStage<NA> st0, st1;
    issue(wave, st0);
    // The columns left out above, while the first group's loads are on their
    // way: wave 0 fetches its 4 rows of A and, value by value, its windows of
    // B (rows outside B as zeros) and adds the column's products to its sums.
    if (wave == 0) {
#pragma clang loop unroll(disable)
        for (int col = 0; col < batch; ++col) {
            if (col == rare_lo) col = rare_hi;
            if (col >= batch) break;
            const unsigned colb = (unsigned)col * ldb4;
            Windows win;
#pragma unroll
            for (int n = 0; n < NWIN; ++n)
#pragma unroll
                for (int q = 0; q < WQ * 4; ++q) {
                    const int r = base + 4 * lane + (n ? delta : 0) + q;
                    win.w[n][q] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                        b_all, (r >= 0 && r < w) ? (unsigned)r * 4u + colb : OOB_OFFSET, 0, 0));
                }
            const __amdgpu_buffer_rsrc_t ar = make_rsrc(A, a_bytes);
            const unsigned cola = (unsigned)col * lda4;
            DdStage<NA> one;
#pragma unroll
            for (int n = 0; n < NA; ++n)
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int r = myrow - (n ? delta : 0) + t;
                    one.a[n][0][t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                        ar, ((r >= 0) & (r < h) & (4 * lane + t < TR)) ? (unsigned)r * 4u + cola : OOB_OFFSET, 0, 0));
                }
            fmas(one, 0, win);
        }
    }
    int k = 0;
    for (; k + 1 < steps; k += 2) {
        step(k, 0, st0, st1);
        step(k + 1, 1, st1, st0);
    }
    if (k < steps) step(k, 0, st0, st1);

    // Combine the waves' partial sums.  8 waves: wave q + 4 hands its sums to
    // wave q first (same lanes, same layout); then the four sums meet in wave
    // order: total = ((p0 + p1) + p2) + p3 with p_q = s_q (+ s_{q+4}).
    __syncthreads();
    float *red = lds;                               // [wave][t][n][j][64 lanes], t blocks RED_T apart
    if (WAVES == 8) {
        if (wave >= 4) {
#pragma unroll
            for (int n = 0; n < NCH; ++n)
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int j = 0; j < LC; ++j)
                        red[(wave - 4) * RED_WAVE + t * RED_T + (n * LC + j) * 64 + lane] = acc[n][t][j];
        }
        __syncthreads();
        if (wave >= 4) return;
#pragma unroll
        for (int n = 0; n < NCH; ++n)
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int j = 0; j < LC; ++j)
                    acc[n][t][j] += red[wave * RED_WAVE + t * RED_T + (n * LC + j) * 64 + lane];
        // no barrier needed here: below, wave q overwrites only the block it has just read
    }
    // (a shifted pair: one chunk after the other through the block of a single chunk)
#pragma unroll
    for (int n0 = 0; n0 < NCH; n0 += NRED) {
        if (n0 > 0) __syncthreads();                // the block is free again
#pragma unroll
        for (int n = 0; n < NRED; ++n)
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int j = 0; j < LC; ++j)
                    red[wave * RED_WAVE + t * RED_T + (n * LC + j) * 64 + lane] = acc[n0 + n][t][j];
        __syncthreads();
        const int r = 64 * wave + lane;             // row within the tile: lane r/4 owned it as its row r%4
        const float *src = red + (r & 3) * RED_T + (r >> 2);
#pragma unroll
        for (int n = 0; n < NRED; ++n)
#pragma unroll
            for (int j = 0; j < LC; ++j) {
                float total = src[(n * LC + j) * 64];
#pragma unroll
                for (int p = 1; p < 4; ++p) total += src[p * RED_WAVE + (n * LC + j) * 64];
                const unsigned off = c_offset(n0 + n, j);
                if (off != OOB_OFFSET) {
                    float *cd = reinterpret_cast<float *>(reinterpret_cast<char *>(C) + off);
                    stream_store(cd, (beta == 0.f) ? alpha * total : beta * cpre[n0 + n][j] + alpha * total);
                }
            }
    }
}

// Shape of the blocks the projection's tiles are numbered in (see the kernel): units per block and row tiles per
// block, 64 positions or nearly.
// Window rows per workgroup (= its waves) of the projection's kernel for rows of 9 to 13 diagonals: 7 (two
// workgroups, 14 waves, per CU) or 5 (three workgroups, 15 waves), whichever leaves fewer wave slots without a window
// row (13 rows -> 7 + 6, 11 -> 7 + 4, 9 -> 5 + 4, 10 -> 5 + 5) -- 5 only where three workgroups' staging buffers fit
// a CU's 160 KB of LDS (two workgroups of 5 waves: 13 x 13 in blocks of 5 took 1.72 ms on the large layer against
// 1.17).  (6 -- 11 rows as 6 + 5 -- measured slower than 7 + 4: two workgroups of 6 waves leave a CU 12 waves.)
// lck: diagonals of a window row; s0: the table's first shift.
inline int dw_long_rows(int k, int lck, int s0)
{
    const int waste5 = (k + 4) / 5 * 5 - k, waste7 = (k + 6) / 7 * 7 - k;
    // the staging buffers of a workgroup of 5 waves (DwLongShape<lck, sh, 5>: 2 buffers of 8 columns)
    const int sh = ((s0 % 4) + 4) % 4, wq = (sh + 4 + lck - 1 + 3) / 4, bpr = 16 + wq - 1;
    const int buf_pieces = (8 * (4 - 1 + 5) * bpr + 63) / 64 * 64 + 8 * 4 * 16;
    const bool three_fit = 3 * 2 * buf_pieces * 16 <= 160 * 1024;
    return waste5 < waste7 && three_fit ? 5 : 7;
}
constexpr int DW_MIN_WGS = 768;               // workgroups from which the window-table projection of a 7 x 7 window is ahead
constexpr int DD_BLOCKED_MIN_TILES = 1024;   // launches of more than a few rounds number their tiles in blocks
struct DdBlock {
    __host__ __device__ static int units(int nunits) { return nunits < 16 ? nunits : 16; }
    __host__ __device__ static int rows(int nunits) { return 64 / units(nunits); }
};

// PAIRS = false: every unit is a single chunk, 4 waves per workgroup.
// PAIRS = true: 8 waves per workgroup; a workgroup whose unit is a single
// chunk retires its upper four waves at once.
template <int LC, bool AVEC, bool PAIRS, int WIDE = DD_NARROW>
__global__ __launch_bounds__((PAIRS && WIDE != DD_SHIFTED) ? 512 : 256) void dd2dia_tiled_kernel(
    const Chunk *__restrict__ chunks, const Unit *__restrict__ units, int nunits,
    float *__restrict__ C, int stride,
    const float *__restrict__ A, long long lda, const float *__restrict__ B, long long ldb,
    int h, int w, int batch, float alpha, float beta, unsigned a_bytes, unsigned b_bytes,
    unsigned c_bytes, int blocked, int h_tiles)
{
    constexpr int NCH_MAX = PAIRS ? 2 : 1;
    static_assert(PAIRS || WIDE == DD_NARROW, "only pairs come in forms");
    constexpr int LDS_FLOATS = dd_lds_floats<LC, NCH_MAX, WIDE>() > dd_lds_floats<LC, 1>() ? dd_lds_floats<LC, NCH_MAX, WIDE>()
                                                                                           : dd_lds_floats<LC, 1>();
    __shared__ __attribute__((aligned(16))) float lds[LDS_FLOATS];
    const int tile = xcd_tile(blockIdx.x, gridDim.x);
    // Tiles are numbered block by block: a block is DdBlock::rows(nunits) neighbouring row tiles x up to 16
    // units, the unit running fastest -- the 64 workgroups an XCD receives together.  The units of a row tile
    // share its 256 rows of A; the unit one window row up of the row tile one period down reads the same band of
    // B: a block of 4 x 16 touches 4 copies of A's rows and about 19 bands where 64 units of one row tile would
    // touch 64 bands.  Positions past the last row tile or unit do nothing.
    // (Launches of one or two rounds keep the plain numbering, unit fastest: every workgroup is resident at
    // once or nearly, and the index arithmetic below -- integer divisions -- would cost them half a microsecond.)
    int rowtile, unit;
    if (!blocked) {
        rowtile = tile / nunits;
        unit = tile - rowtile * nunits;
    } else {
    const int ub = DdBlock::units(nunits), rb = DdBlock::rows(nunits), nub = (nunits + ub - 1) / ub;
    const int per_rblk = nub * rb * ub;
    const int rblk = tile / per_rblk, rem = tile - rblk * per_rblk;
    // Workgroup ids go to the XCDs round-robin by spans of 64: with the unit blocks of a row block always in the
    // same order an XCD would meet the same unit block again and again -- and the unit blocks of a multi-channel
    // table differ in how many of their units lie inside the operand.  The order is therefore turned by one
    // place every time the spans have gone round the XCDs.
    const int turn = rblk / (nub < 8 ? 8 / nub : 1);
    const int ublk = (rem / (rb * ub) + turn) % nub, pos = rem % (rb * ub);
    rowtile = rblk * rb + pos / ub;
    unit = ublk * ub + pos % ub;
    }
    constexpr int TR = (PAIRS && WIDE != DD_SHIFTED) ? DD_ROWS : dd_short_rows<LC>();        // rows of a tile
    // h_tiles: row tiles of the launch -- those of A's rows, and for shifted pairs the tiles past them whose second
    // chunk still works on rows of A
    if (rowtile >= h_tiles || unit >= nunits) return;
    typedef const Unit __attribute__((address_space(4))) *sc_unit_ptr;
    const sc_unit_ptr u = (sc_unit_ptr)units + unit;
    const int c1 = u->c1, c2 = u->c2;
    const int row0 = rowtile * TR;
    if constexpr (PAIRS) {
        if (c2 >= 0) {
            dd2dia_unit<LC, 2, AVEC, WIDE>(lds, row0, chunks + c1, chunks + c2, C, stride, A, lda, B, ldb, h, w, batch,
                                           alpha, beta, a_bytes, b_bytes, c_bytes);
            return;
        }
    }
    if (PAIRS && threadIdx.x >= 256) return;
    if (row0 >= h) return;
    dd2dia_unit<LC, 1, AVEC, DD_NARROW, !PAIRS || WIDE == DD_SHIFTED>(lds, row0, chunks + c1, chunks + c1, C, stride, A, lda, B, ldb, h, w, batch,
                             alpha, beta, a_bytes, b_bytes, c_bytes);
}

// ------------------------------------------------------- window-table dd2dia --
//
// The projection for *window* tables (plan_walk: k window rows `period` rows apart, every chunk LC <= 8 shifts,
// repeated for every group), tiled in the plane the window lives in.  Row i of A is position (y, x) =
// (i / period, i mod period); slot (dy, j) of group g pairs it with row i + s0 + group_rows[g] + dy * period + j of
// B.  A workgroup owns a tile of 4 x 64 positions -- wave = one y, 64 consecutive x -- for up to 8 window rows
// (DYB; a taller window is served by several workgroups per tile) and walks the batch in groups of 4 columns.
// Per group it stages, with loads that write LDS directly,
//   * its 4 x 64 values of A per column (16 pieces of 16 bytes per y), and
//   * the 4 + rows - 1 stretches of B that its window rows reach, 64 + SH + LC - 1 values each (BPR pieces),
// each value ONCE for all the slots that use it: (256 + 10 * 72) * 4 B per column for 49 * 256 FMAs of a 7 x 7
// window, a third of what 256 rows cost the chunk-by-chunk kernel above (3 KB per 14 * 248 FMAs).  The stretches
// start at the multiple of 4 at or below their first row (SH = s0 mod 4, the same for every group: a template
// parameter, so a lane's window keeps static register indices); with row counts that are multiples of 4 every
// 16-byte piece lies wholly inside its column or outside, and the pieces outside are requested out of range and
// arrive as zeros.
// Lane = (role r = lane / 16, xg = lane mod 16): positions x = 64 tx + 4 xg .. + 3 of the wave's y, window rows
// dy = 2r and 2r + 1 of the workgroup's eight: 2 x 4 x LC running sums, one 16-byte read of A and two windows
// of B (4 + LC - 1 values each, WQ 16-byte reads) per column.  A ring of NBUF LDS buffers: while group i is
// applied, the groups up to i + NBUF - 1 land; one wait and one barrier per group.  (Two buffers of 4 columns
// measured best: with 4 buffers of 2 columns -- half as much again in flight in the same LDS -- the 512 x 512
// map at batch 512 took 344 us instead of 315, with 3 buffers of 4 columns, which leave room for 2 or 3
// workgroups per CU, 424.  What bounds the kernel at those sizes is the operands' one trip from memory:
// with neither FMAs nor LDS reads it takes 288 us.)  A lane's share of a group's requests is the same for the
// whole walk up to the column step, so its byte offsets are computed once; everything, column included, goes
// into the vector offset, which the buffer's range check covers.
//
// Accumulation order per slot: batch columns ascending, acc = fma(a, b, acc); C = beta*C + alpha*acc.  With
// SUBS batch ranges per workgroup (see the kernel): p_r over range r's columns ascending, then
// acc = ((p_0 + p_1) + p_2) + p_3.
template <int LC, int SH>
struct DwShape {
    static constexpr int WAVES = 4, TX = 64, DYB = 8;
    static constexpr int COLS = 4;                               // batch columns per staged group
    static constexpr int NBUF = 2;                               // LDS buffers: the group applied + those in flight
    static constexpr int WIN = SH + 4 + LC - 1;                  // values of a lane's window, from its first piece
    static constexpr int WQ = (WIN + 3) / 4;                     // .. as 16-byte reads
    static constexpr int BPR = TX / 4 + WQ - 1;                  // pieces per staged stretch of B
    static constexpr int NBR_MAX = WAVES - 1 + DYB;              // stretches per column
    static constexpr int B_PIECES = (COLS * NBR_MAX * BPR + 63) / 64 * 64;
    static constexpr int A_PIECES = COLS * WAVES * (TX / 4);
    static constexpr int BUF_PIECES = B_PIECES + A_PIECES;
    static constexpr int NI_MAX = BUF_PIECES / 64;               // load instructions per group
    static constexpr int NIT = (NI_MAX + WAVES - 1) / WAVES;     // .. per wave
    static_assert(A_PIECES % 64 == 0 && LC >= 1 && LC <= CHUNK_MAX && SH >= 0 && SH < 4, "shape");
    static_assert(NBUF >= 2 && NBUF * BUF_PIECES * 16 <= 40 * 1024, "four workgroups share a CU's LDS");
    static_assert((NBUF - 2) * NIT <= 8, "the waits name up to eight requests left in flight");
};

// calls body(gi + I, I) for I = 0 .. N-1 while gi + I < n: the position in the ring is a compile-time constant
template <int N, int I, class F>
__device__ __forceinline__ void dw_ring(F &body, int gi, int n)
{
    if constexpr (I < N) {
        if (gi + I < n) body(gi + I, std::integral_constant<int, I>{});
        dw_ring<N, I + 1>(body, gi, n);
    }
}

// SUBS: the batch is cut into SUBS ranges of whole groups, each worked by 4 of the workgroup's 4 x SUBS waves with
// staging buffers of their own (launches of few tiles: 2 or 4 ranges keep 16 waves on every CU where one
// range per tile would leave most of the chip idle).  The ranges' sums meet in LDS at the end, in range order.
template <int LC, int SH, int SUBS>
__global__ __launch_bounds__(256 * SUBS, 4) void dd2dia_window_kernel(
    const int *__restrict__ tab,            // group_rows[ngroups], then 4 * element offset of chunk (g, dy)'s first slot
    int ngroups, int K, int period, int s0, int astep, float *__restrict__ C,
    const float *__restrict__ A, long long lda, const float *__restrict__ B, long long ldb,
    int h, int w, int batch, float alpha, float beta, unsigned a_bytes, unsigned b_bytes, unsigned c_bytes,
    int txn, int tyn, int ndb)
{
    typedef DwShape<LC, SH> S;
    constexpr int WAVES = S::WAVES, COLS = S::COLS, DYB = S::DYB, WQ = S::WQ, BPR = S::BPR, NIT = S::NIT;
    static_assert(SUBS == 1 || SUBS == 2 || SUBS == 4, "batch ranges per workgroup");
    __shared__ __attribute__((aligned(16))) float lds_all[SUBS][S::NBUF][S::BUF_PIECES * 4];
    static_assert((SUBS - 1) * WAVES * 4 * LC * 64 <= SUBS * S::NBUF * S::BUF_PIECES * 4, "the ranges' sums fit the staging buffers");
    const int lane = threadIdx.x & 63;
    const int wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int sub = wave_all / WAVES, wave = wave_all % WAVES;      // batch range, wave within it
    float (*lds)[S::BUF_PIECES * 4] = lds_all[sub];
    typedef const int __attribute__((address_space(4))) *sc_int_ptr;
    const sc_int_ptr stab = (sc_int_ptr)tab;

    // workgroup -> (group, tile row, block of window rows, tile column), the tile column fastest: the 64
    // workgroups an XCD receives together are a band of neighbouring tiles, which share their stretches of B, and
    // the blocks of a tall window sit side by side, where they find the tile's rows of A in the L2
    int rest = xcd_tile(blockIdx.x, gridDim.x);
    const int tx = rest % txn; rest /= txn;
    const int db = rest % ndb; rest /= ndb;
    const int ty = rest % tyn;
    const int g = rest / tyn;
    const int kb = min(DYB, K - DYB * db);                    // window rows served here
    const int nbr = WAVES - 1 + kb;                           // stretches of B per column
    const int i_tile = 4 * ty * period + S::TX * tx;          // the tile's first row of A
    const int s_g = s0 + stab[g] + DYB * db * period;         // shift of this block's first slot
    const int b_tile = i_tile + s_g - SH;                     // first staged row of B, a multiple of 4
    // every slot of the workgroup pairs rows of A with rows [b_tile, b_hi) of B: nothing to do when none exists
    const int b_hi = b_tile + (nbr - 1) * period + 4 * BPR;
    if (i_tile >= h || b_hi <= 0 || b_tile >= w) return;

    // This lane's requests of a group: instruction s = wave + WAVES * it carries pieces 64 s .. 64 s + 63 of the
    // buffer -- B's first ((column, stretch, piece), nib instructions), then A's ((column, y, piece)).
    const int npb = COLS * nbr * BPR;
    const int nib = (npb + 63) / 64;
    const int ni = nib + S::A_PIECES / 64;
    // groups per batch range (the same for every range: a range that ends past the batch works on zeros there)
    const int ngr = ((batch + COLS - 1) / COLS + SUBS - 1) / SUBS;
    const int col_first = sub * ngr * COLS;
    unsigned v_lane[NIT];
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
        const int s = wave + WAVES * it;
        unsigned v = OOB_OFFSET;
        if (s < nib) {
            const int p = 64 * s + lane;
            const int col = p / (nbr * BPR), rem = p - col * (nbr * BPR);
            const int row = rem / BPR, pc = rem - row * BPR;
            const int idx = b_tile + row * period + 4 * pc;
            // (64-bit: a column past the batch may lie past 2^31 bytes; it is out of range either way)
            const long long at = ((long long)(col_first + col) * ldb + idx) * 4;
            if ((p < npb) & (idx >= 0) & (idx + 4 <= w) & (at < (long long)OOB_OFFSET)) v = (unsigned)at;
        } else if (s < ni) {
            const int col = s - nib, row = lane >> 4, pc = lane & 15;
            const int idx = i_tile + row * period + 4 * pc;
            const long long at = ((long long)(col_first + col) * lda + idx) * 4;
            if ((idx + 4 <= h) & (at < (long long)OOB_OFFSET)) v = (unsigned)at;
        }
        v_lane[it] = v;
    }
    const sp_int4 bq = raw_rsrc(B, b_bytes), aq = raw_rsrc(A, a_bytes);
    const unsigned lds0 = (unsigned)(unsigned long long)(__attribute__((address_space(3))) float *)&lds_all[0][0][0] +
                          (unsigned)sub * (S::NBUF * S::BUF_PIECES * 16u);
    constexpr unsigned BUF_BYTES = S::BUF_PIECES * 16u;
    const unsigned b_step = (unsigned)ldb * (4u * COLS), a_step = (unsigned)lda * (4u * COLS);    // bytes per group
    // Requests the next group into buffer `par` and moves the lane's offsets one group on.  (An offset that is
    // out of range stays so: it starts at 2^31, and all the steps of a walk add up to less than an operand's size.)
    auto issue = [&](int par) __attribute__((always_inline)) {
        const unsigned buf = lds0 + (unsigned)par * BUF_BYTES;
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const int s = wave + WAVES * it;
            if (s < nib) {
                lds_load_b128(bq, buf + 1024u * (unsigned)s, v_lane[it], 0u);
                v_lane[it] += b_step;
            } else if (s < ni) {
                lds_load_b128(aq, buf + (unsigned)S::B_PIECES * 16u + 1024u * (unsigned)(s - nib), v_lane[it], 0u);
                v_lane[it] += a_step;
            }
        }
    };

    const int role = lane >> 4, xg = lane & 15;
    // floats from a buffer's start to this lane's windows (column 0) and to its piece of A
    int w_off[2];
#pragma unroll
    for (int n = 0; n < 2; ++n) w_off[n] = ((wave + min(2 * role + n, kb - 1)) * BPR + xg) * 4;
    const int col_floats = nbr * BPR * 4;
    const int a_off = S::B_PIECES * 4 + (wave * 16 + xg) * 4;

    float acc[2][4][LC];
#pragma unroll
    for (int n = 0; n < 2; ++n)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int j = 0; j < LC; ++j) acc[n][t][j] = 0.f;

    typedef float v4f __attribute__((ext_vector_type(4)));
    struct Win { v4f p[WQ]; };
    auto read_win = [&](Win &win, const float *buf, int c, int n) __attribute__((always_inline)) {
        const v4f *p4 = reinterpret_cast<const v4f *>(buf + c * col_floats + w_off[n]);
#pragma unroll
        for (int q = 0; q < WQ; ++q) win.p[q] = p4[q];
    };
    auto fmas = [&](int n, const float4 &a, Win &win) __attribute__((always_inline)) {
        const float av[4] = {a.x, a.y, a.z, a.w};
        float wv[WQ * 4];
#pragma unroll
        for (int q = 0; q < WQ; ++q) {
            // (The window's first and last values may be unused: without this the compiler fetches the others one
            // by one, and four-byte reads 16 bytes apart share their banks four ways.  The asm sits where the
            // window is used, not where it is read: the wait for the read goes with it.)
            v4f v = win.p[q];
            asm volatile("" : "+v"(v));
            wv[4 * q + 0] = v.x; wv[4 * q + 1] = v.y; wv[4 * q + 2] = v.z; wv[4 * q + 3] = v.w;
        }
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int j = 0; j < LC; ++j) acc[n][t][j] = __builtin_fmaf(av[t], wv[SH + t + j], acc[n][t][j]);
    };
    // One group: the second window of a column and the next column's first are read while the FMAs of the
    // window before them run.
    auto apply = [&](const float *buf) __attribute__((always_inline)) {
        Win w0, w1;
        float4 a0, a1;
        a0 = *reinterpret_cast<const float4 *>(buf + a_off);
        read_win(w0, buf, 0, 0);
#pragma unroll
        for (int c = 0; c < COLS; ++c) {
            float4 &ac = (c & 1) ? a1 : a0;
            float4 &an = (c & 1) ? a0 : a1;
            read_win(w1, buf, c, 1);
            __builtin_amdgcn_sched_barrier(0);
            fmas(0, ac, w0);
            __builtin_amdgcn_sched_barrier(0);
            if (c + 1 < COLS) {
                an = *reinterpret_cast<const float4 *>(buf + a_off + (c + 1) * 256);
                read_win(w0, buf, c + 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            fmas(1, ac, w1);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // The ring: group gi is applied out of buffer gi mod NBUF while the groups up to gi + NBUF - 1 are in flight or
    // landed.  At a group's end everything but the requests of the groups after the next has to have arrived: this
    // wave's share of a group is n_mine instructions, and they complete in order.
    // (columns past the batch start a whole column past the last one: out of the resources' range, they arrive
    // as zeros and add nothing)
    const int n_mine = (ni - wave + WAVES - 1) / WAVES;
    auto wait_leaving_groups = [&](int groups) __attribute__((always_inline)) {
        switch (groups * n_mine) {
            case 0: asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); break;
            case 1: asm volatile("s_waitcnt vmcnt(1) lgkmcnt(0)" ::: "memory"); break;
            case 2: asm volatile("s_waitcnt vmcnt(2) lgkmcnt(0)" ::: "memory"); break;
            case 3: asm volatile("s_waitcnt vmcnt(3) lgkmcnt(0)" ::: "memory"); break;
            case 4: asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory"); break;
            case 5: asm volatile("s_waitcnt vmcnt(5) lgkmcnt(0)" ::: "memory"); break;
            case 6: asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)" ::: "memory"); break;
            case 7: asm volatile("s_waitcnt vmcnt(7) lgkmcnt(0)" ::: "memory"); break;
            default: asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory"); break;
        }
    };
    constexpr int NBUF = S::NBUF;
    for (int k = 0; k < NBUF - 1; ++k)
        if (k < ngr) issue(k);
    wait_leaving_groups(min(NBUF - 2, ngr - 1));
    __syncthreads();
    auto body = [&](int gi, auto cur_c) __attribute__((always_inline)) {
        constexpr int cur = decltype(cur_c)::value;
        // (the buffer the group before this one was applied from: every wave left it at the last barrier)
        if (gi + NBUF - 1 < ngr) issue((cur + NBUF - 1) % NBUF);
        apply(&lds[cur][0]);
        wait_leaving_groups(max(0, min(NBUF - 2, ngr - 2 - gi)));
        __syncthreads();
    };
#pragma clang loop unroll(disable)
    for (int gi = 0; gi < ngr; gi += NBUF) dw_ring<NBUF, 0>(body, gi, ngr);

    // The ranges' sums meet: half of them at a time (one of a lane's two window rows), ranges 1 .. SUBS - 1 write,
    // range 0 adds them in range order.  (Every wave has passed the loop's last barrier: the buffers are free.)
    if constexpr (SUBS > 1) {
        float *red = &lds_all[0][0][0];
        constexpr int PER_WAVE = 4 * LC * 64;
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            if (sub > 0) {
                float *dst = red + ((sub - 1) * WAVES + wave) * PER_WAVE + lane;
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int j = 0; j < LC; ++j) dst[(t * LC + j) * 64] = acc[n][t][j];
            }
            __syncthreads();
            if (sub == 0) {
#pragma unroll
                for (int r = 1; r < SUBS; ++r) {
                    const float *src = red + ((r - 1) * WAVES + wave) * PER_WAVE + lane;
#pragma unroll
                    for (int t = 0; t < 4; ++t)
#pragma unroll
                        for (int j = 0; j < LC; ++j) acc[n][t][j] += src[(t * LC + j) * 64];
                }
            }
            __syncthreads();
        }
        if (sub > 0) return;
    }

    // Results: 4 consecutive rows of every slot per lane, one 16-byte store where all four exist.
    typedef float f4u __attribute__((ext_vector_type(4), aligned(4)));
    typedef unsigned sp_u4 __attribute__((ext_vector_type(4)));
    const __amdgpu_buffer_rsrc_t cr = make_rsrc(C, c_bytes);
    const int o = i_tile + wave * period + 4 * xg;              // the lane's first row of A
    const bool x_ok = S::TX * tx + 4 * xg < period;             // (a narrower last tile column: the positions past the
                                                                // row belong to the next row's first tile)
    // (A window row's old values are all requested before the first of them is used: a request per slot, waited
    // for and stored before the next, cost the workgroup LC round trips to memory in a row.)
#pragma unroll
    for (int n = 0; n < 2; ++n) {
        const int dyl = 2 * role + n;
        const bool dy_ok = dyl < kb;
        const int dy = DYB * db + (dy_ok ? dyl : 0);
        const int e0 = tab[ngroups + g * K + dy] / 4 + o;       // element of slot j = 0 for row o
        const int in0 = o + s_g + dyl * period;                 // the row of B that row o meets in slot j = 0
        unsigned off[LC], okbits[LC];
        f4u old4[LC];
        bool any_part = false;                                  // wave-uniform: some lane has a partly valid group of 4
#pragma unroll
        for (int j = 0; j < LC; ++j) {
            unsigned bits = 0;
#pragma unroll
            for (int t = 0; t < 4; ++t)
                bits |= (unsigned)(dy_ok & x_ok & (o + t < h) & ((unsigned)(in0 + j + t) < (unsigned)w)) << t;
            okbits[j] = bits;
            off[j] = (unsigned)(e0 + j * astep) * 4u;
            any_part = any_part || __builtin_amdgcn_ballot_w64(bits != 0u && bits != 15u) != 0ull;
            old4[j] = f4u{0.f, 0.f, 0.f, 0.f};
            if (beta != 0.f)
                old4[j] = __builtin_bit_cast(f4u, __builtin_amdgcn_raw_buffer_load_b128(cr, bits == 15u ? off[j] : OOB_OFFSET, 0, 0));
        }
        if (!any_part) {
            // every lane's groups of 4 are whole or empty: nothing but the stores, no wait between them
#pragma unroll
            for (int j = 0; j < LC; ++j) {
                float r[4];
                const float old[4] = {old4[j].x, old4[j].y, old4[j].z, old4[j].w};
#pragma unroll
                for (int t = 0; t < 4; ++t) r[t] = (beta == 0.f) ? alpha * acc[n][t][j] : beta * old[t] + alpha * acc[n][t][j];
                __builtin_amdgcn_raw_buffer_store_b128(sp_u4{__builtin_bit_cast(unsigned, r[0]), __builtin_bit_cast(unsigned, r[1]),
                                                             __builtin_bit_cast(unsigned, r[2]), __builtin_bit_cast(unsigned, r[3])},
                                                       cr, okbits[j] == 15u ? off[j] : OOB_OFFSET, 0, 2);
            }
        } else {
            // workgroups at the matrix's first and last rows: the partly valid groups row by row
#pragma unroll
            for (int j = 0; j < LC; ++j) {
                const bool all4 = okbits[j] == 15u;
                const bool part = okbits[j] != 0u && !all4;
                float old[4] = {old4[j].x, old4[j].y, old4[j].z, old4[j].w};
                if (beta != 0.f) {
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const float v = buffer_load_f32(cr, (part && ((okbits[j] >> t) & 1u)) ? off[j] + 4u * t : OOB_OFFSET);
                        old[t] = part ? v : old[t];
                    }
                }
                float r[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) r[t] = (beta == 0.f) ? alpha * acc[n][t][j] : beta * old[t] + alpha * acc[n][t][j];
                __builtin_amdgcn_raw_buffer_store_b128(sp_u4{__builtin_bit_cast(unsigned, r[0]), __builtin_bit_cast(unsigned, r[1]),
                                                             __builtin_bit_cast(unsigned, r[2]), __builtin_bit_cast(unsigned, r[3])},
                                                       cr, all4 ? off[j] : OOB_OFFSET, 0, 2);
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, r[t]), cr,
                                                          (part && ((okbits[j] >> t) & 1u)) ? off[j] + 4u * t : OOB_OFFSET, 0, 2);
            }
        }
    }
}

// The same tiling for window rows of 9 to 13 diagonals (a chunk of the products' table: the large layer's 13 x 13
// window), with the roles turned round: a wave's 2 x 4 x LC sums would not fit its registers, so here a WAVE owns
// one window row (5 or 7 of them per workgroup, dw_long_rows; a taller window takes several workgroups per tile) and
// a lane's role is the y of the tile's four: 4 x LC running sums, one 16-byte read of A and one window of B
// (4 + LC - 1 values) per column.  Staging, ring, waits and the results' way out are those of the kernel above; a
// wave past the block's last window row only helps with the requests.
template <int LC, int SH, int NW>
struct DwLongShape {
    static constexpr int WAVES = NW, YT = 4, TX = 64;
    static constexpr int COLS = 8;                               // batch columns per staged group
    static constexpr int NBUF = 2;                               // (3 or 4 buffers of 4 columns measured 3 - 4 % slower)
    static constexpr int WIN = SH + 4 + LC - 1;
    static constexpr int WQ = (WIN + 3) / 4;
    static constexpr int BPR = TX / 4 + WQ - 1;
    static constexpr int NBR_MAX = YT - 1 + WAVES;
    static constexpr int B_PIECES = (COLS * NBR_MAX * BPR + 63) / 64 * 64;
    static constexpr int A_PIECES = COLS * YT * (TX / 4);
    static constexpr int BUF_PIECES = B_PIECES + A_PIECES;
    static constexpr int NI_MAX = BUF_PIECES / 64;
    static constexpr int NIT = (NI_MAX + WAVES - 1) / WAVES;
    static_assert(A_PIECES % 64 == 0 && LC > CHUNK_MAX && LC <= SP_CHUNK_MAX && SH >= 0 && SH < 4, "shape");
    static_assert(NBUF >= 2 && NBUF * BUF_PIECES * 16 <= 80 * 1024, "two buffers; two workgroups per CU and to spare");
};

template <int LC, int SH, int NW>
__global__ __launch_bounds__(64 * NW, 4) void dd2dia_window_long_kernel(
    const int *__restrict__ tab, int ngroups, int K, int period, int s0, int astep, float *__restrict__ C,
    const float *__restrict__ A, long long lda, const float *__restrict__ B, long long ldb,
    int h, int w, int batch, float alpha, float beta, unsigned a_bytes, unsigned b_bytes, unsigned c_bytes,
    int txn, int tyn, int ndb)
{
    typedef DwLongShape<LC, SH, NW> S;
    static_assert(NW == 5 || NW == 7, "waves per workgroup");
    static_assert(S::COLS == 8 && S::NBUF == 2 && S::YT == 4 && S::TX == 64, "dw_long_rows computes the buffers' size from these");
    constexpr int WAVES = S::WAVES, YT = S::YT, COLS = S::COLS, WQ = S::WQ, BPR = S::BPR, NIT = S::NIT;
    __shared__ __attribute__((aligned(16))) float lds[S::NBUF][S::BUF_PIECES * 4];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    typedef const int __attribute__((address_space(4))) *sc_int_ptr;
    const sc_int_ptr stab = (sc_int_ptr)tab;

    // workgroup -> (group, tile row, block of window rows, tile column): the blocks of a tile side by side, so that
    // they find the tile's rows of A and the stretches they share in the XCD's L2
    int rest = xcd_tile(blockIdx.x, gridDim.x);
    const int tx = rest % txn; rest /= txn;
    const int db = rest % ndb; rest /= ndb;
    const int ty = rest % tyn;
    const int g = rest / tyn;
    const int kb = min(WAVES, K - WAVES * db);                // window rows served here
    const int nbr = YT - 1 + kb;                              // stretches of B per column
    const int i_tile = YT * ty * period + S::TX * tx;         // the tile's first row of A
    const int s_g = s0 + stab[g] + WAVES * db * period;       // shift of this block's first slot
    const int b_tile = i_tile + s_g - SH;                     // first staged row of B, a multiple of 4
    const int b_hi = b_tile + (nbr - 1) * period + 4 * BPR;
    if (i_tile >= h || b_hi <= 0 || b_tile >= w) return;

    const int npb = COLS * nbr * BPR;
    const int nib = (npb + 63) / 64;
    const int ni = nib + S::A_PIECES / 64;
    const int ngr = (batch + COLS - 1) / COLS;
    unsigned v_lane[NIT];
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
        const int s = wave + WAVES * it;
        unsigned v = OOB_OFFSET;
        if (s < nib) {
            const int p = 64 * s + lane;
            const int col = p / (nbr * BPR), rem = p - col * (nbr * BPR);
            const int row = rem / BPR, pc = rem - row * BPR;
            const int idx = b_tile + row * period + 4 * pc;
            const long long at = ((long long)col * ldb + idx) * 4;
            if ((p < npb) & (idx >= 0) & (idx + 4 <= w) & (at < (long long)OOB_OFFSET)) v = (unsigned)at;
        } else if (s < ni) {
            const int col = s - nib, row = lane >> 4, pc = lane & 15;
            const int idx = i_tile + row * period + 4 * pc;
            const long long at = ((long long)col * lda + idx) * 4;
            if ((idx + 4 <= h) & (at < (long long)OOB_OFFSET)) v = (unsigned)at;
        }
        v_lane[it] = v;
    }
    const sp_int4 bq = raw_rsrc(B, b_bytes), aq = raw_rsrc(A, a_bytes);
    const unsigned lds0 = (unsigned)(unsigned long long)(__attribute__((address_space(3))) float *)&lds[0][0];
    constexpr unsigned BUF_BYTES = S::BUF_PIECES * 16u;
    const unsigned b_step = (unsigned)ldb * (4u * COLS), a_step = (unsigned)lda * (4u * COLS);
    auto issue = [&](int par) __attribute__((always_inline)) {
        const unsigned buf = lds0 + (unsigned)par * BUF_BYTES;
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const int s = wave + WAVES * it;
            if (s < nib) {
                lds_load_b128(bq, buf + 1024u * (unsigned)s, v_lane[it], 0u);
                v_lane[it] += b_step;
            } else if (s < ni) {
                lds_load_b128(aq, buf + (unsigned)S::B_PIECES * 16u + 1024u * (unsigned)(s - nib), v_lane[it], 0u);
                v_lane[it] += a_step;
            }
        }
    };

    const int role = lane >> 4, xg = lane & 15;               // role = the lane's y of the tile's four
    const bool active = wave < kb;                            // (wave-uniform)
    const int w_off = ((role + min(wave, kb - 1)) * BPR + xg) * 4;
    const int col_floats = nbr * BPR * 4;
    const int a_off = S::B_PIECES * 4 + (role * 16 + xg) * 4;

    float acc[4][LC];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int j = 0; j < LC; ++j) acc[t][j] = 0.f;

    // One group.  A column's FMAs run in the order of the window values they use; as soon as a 16-byte piece of the
    // window has served its last FMA, the same registers take the next column's piece -- one window in registers,
    // its reads hidden behind the FMAs of the pieces after it.
    // (The pieces stay whole 16-byte reads because each passes through an empty asm -- see the kernel above -- and
    // that asm sits where the piece is first used, not where it is read: the wait for the read goes with it.)
    typedef float v4f __attribute__((ext_vector_type(4)));
    v4f wv[WQ];
    auto read_piece = [&](const float *buf, int c, int q) __attribute__((always_inline)) {
        wv[q] = reinterpret_cast<const v4f *>(buf + c * col_floats + w_off)[q];
    };
    auto apply = [&](const float *buf) __attribute__((always_inline)) {
        float4 a0, a1;
        a0 = *reinterpret_cast<const float4 *>(buf + a_off);
#pragma unroll
        for (int q = 0; q < WQ; ++q) read_piece(buf, 0, q);
#pragma unroll
        for (int c = 0; c < COLS; ++c) {
            float4 &ac = (c & 1) ? a1 : a0;
            float4 &an = (c & 1) ? a0 : a1;
            if (c + 1 < COLS) an = *reinterpret_cast<const float4 *>(buf + a_off + (c + 1) * 256);
            const float av[4] = {ac.x, ac.y, ac.z, ac.w};
#pragma unroll
            for (int q = 0; q < WQ; ++q) {
                __builtin_amdgcn_sched_barrier(0);
                v4f v = wv[q];
                asm volatile("" : "+v"(v));
                const float win4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const int j = 4 * q + e - SH - t;
                        if (j >= 0 && j < LC) acc[t][j] = __builtin_fmaf(av[t], win4[e], acc[t][j]);
                    }
                __builtin_amdgcn_sched_barrier(0);
                if (c + 1 < COLS) read_piece(buf, c + 1, q);
            }
        }
    };

    // The ring (as in the kernel above): group gi is applied out of buffer gi mod NBUF while the groups up to
    // gi + NBUF - 1 are in flight or landed; at a group's end everything but the requests of the groups after the
    // next has to have arrived -- this wave's share of a group is n_mine instructions, and they complete in order.
    constexpr int NBUF = S::NBUF;
    const int n_mine = (ni - wave + WAVES - 1) / WAVES;
    auto wait_leaving_groups = [&](int groups) __attribute__((always_inline)) {
        switch (groups * n_mine) {
            case 0: asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); break;
            case 1: asm volatile("s_waitcnt vmcnt(1) lgkmcnt(0)" ::: "memory"); break;
            case 2: asm volatile("s_waitcnt vmcnt(2) lgkmcnt(0)" ::: "memory"); break;
            case 3: asm volatile("s_waitcnt vmcnt(3) lgkmcnt(0)" ::: "memory"); break;
            case 4: asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory"); break;
            case 5: asm volatile("s_waitcnt vmcnt(5) lgkmcnt(0)" ::: "memory"); break;
            case 6: asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)" ::: "memory"); break;
            case 7: asm volatile("s_waitcnt vmcnt(7) lgkmcnt(0)" ::: "memory"); break;
            default: asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory"); break;
        }
    };
    static_assert((NBUF - 2) * NIT <= 8, "the waits name up to eight requests left in flight");
    for (int k = 0; k < NBUF - 1; ++k)
        if (k < ngr) issue(k);
    wait_leaving_groups(min(NBUF - 2, ngr - 1));
    __syncthreads();
    auto body = [&](int gi, auto cur_c) __attribute__((always_inline)) {
        constexpr int cur = decltype(cur_c)::value;
        if (gi + NBUF - 1 < ngr) issue((cur + NBUF - 1) % NBUF);
        if (active) apply(&lds[cur][0]);
        wait_leaving_groups(max(0, min(NBUF - 2, ngr - 2 - gi)));
        __syncthreads();
    };
#pragma clang loop unroll(disable)
    for (int gi = 0; gi < ngr; gi += NBUF) dw_ring<NBUF, 0>(body, gi, ngr);
    if (!active) return;

    // Results: 4 consecutive rows of every slot of the wave's window row per lane.
    typedef float f4u __attribute__((ext_vector_type(4), aligned(4)));
    typedef unsigned sp_u4 __attribute__((ext_vector_type(4)));
    const __amdgpu_buffer_rsrc_t cr = make_rsrc(C, c_bytes);
    const int o = i_tile + role * period + 4 * xg;              // the lane's first row of A
    const bool x_ok = S::TX * tx + 4 * xg < period;
    const int dy = WAVES * db + wave;
    const int e0 = tab[ngroups + g * K + dy] / 4 + o;           // element of slot j = 0 for row o
    const int in0 = o + s_g + wave * period;                    // the row of B that row o meets in slot j = 0
    // (half of the window row's slots at a time: their old values, requested together, and the sums share the
    // registers)
    constexpr int JH = (LC + 1) / 2;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const int j0 = half * JH;
        unsigned off[JH], okbits[JH];
        f4u old4[JH];
        bool any_part = false;
#pragma unroll
        for (int jj = 0; jj < JH; ++jj) {
            const int j = j0 + jj;
            unsigned bits = 0;
            if (j < LC) {
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    bits |= (unsigned)(x_ok & (o + t < h) & ((unsigned)(in0 + j + t) < (unsigned)w)) << t;
            }
            okbits[jj] = bits;
            off[jj] = (unsigned)(e0 + j * astep) * 4u;
            any_part = any_part || __builtin_amdgcn_ballot_w64(bits != 0u && bits != 15u) != 0ull;
            old4[jj] = f4u{0.f, 0.f, 0.f, 0.f};
            if (beta != 0.f)
                old4[jj] = __builtin_bit_cast(f4u, __builtin_amdgcn_raw_buffer_load_b128(cr, bits == 15u ? off[jj] : OOB_OFFSET, 0, 0));
        }
#pragma unroll
        for (int jj = 0; jj < JH; ++jj) {
            const int j = j0 + jj;
            if (j >= LC) continue;
            const bool all4 = okbits[jj] == 15u;
            const bool part = okbits[jj] != 0u && !all4;
            float old[4] = {old4[jj].x, old4[jj].y, old4[jj].z, old4[jj].w};
            if (any_part && beta != 0.f) {
                // workgroups at the matrix's first and last rows: the partly valid groups row by row
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const float v = buffer_load_f32(cr, (part && ((okbits[jj] >> t) & 1u)) ? off[jj] + 4u * t : OOB_OFFSET);
                    old[t] = part ? v : old[t];
                }
            }
            float r[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) r[t] = (beta == 0.f) ? alpha * acc[t][j] : beta * old[t] + alpha * acc[t][j];
            __builtin_amdgcn_raw_buffer_store_b128(sp_u4{__builtin_bit_cast(unsigned, r[0]), __builtin_bit_cast(unsigned, r[1]),
                                                         __builtin_bit_cast(unsigned, r[2]), __builtin_bit_cast(unsigned, r[3])},
                                                   cr, all4 ? off[jj] : OOB_OFFSET, 0, 2);
            if (any_part) {
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, r[t]), cr,
                                                          (part && ((okbits[jj] >> t) & 1u)) ? off[jj] + 4u * t : OOB_OFFSET, 0, 2);
            }
        }
    }
}

}  // namespace

// ---------------------------------------------------------------- launchers --

#if CUVDIA_IN_PART(4)
hipError_t launch_spmm_generic(const DiaView &A, const float *vals, const float *B, long long ldb,
                               float *dst, long long ldd, int batch, bool trans,
                               float alpha, float beta, SpEpilogue ep, hipStream_t stream)
{
    const int n_out = trans ? A.w : A.h;
    constexpr int CB = 4;
    const unsigned gx = (unsigned)((n_out + 255) / 256);
    int done = 0;
    // grid.y is limited to 65535: walk very wide batches in slabs
    while (done < batch) {
        const int slab = batch - done < 65535 * CB ? batch - done : 65535 * CB;
        const dim3 grid(gx, (unsigned)((slab + CB - 1) / CB));
        note_kernel("spmm_generic_kernel<%d>", CB);
        hipLaunchKernelGGL(spmm_generic_kernel<CB>, grid, dim3(256), 0, stream,
                           A.offsets_dev, A.nd, vals, A.stride, A.h, A.w, A.rf,
                           B + (long long)done * ldb, ldb, dst + (long long)done * ldd, ldd,
                           n_out, slab, trans ? 1 : 0, alpha, beta, ep);
        done += slab;
    }
    return hipGetLastError();
}

bool spmm_tiled_ok(const DiaView &A, long long ldb, long long ldd, bool trans)
{
    // buffer resources address 32-bit byte offsets below the out-of-range marker
    const long long n_in = trans ? A.h : A.w, n_out = trans ? A.w : A.h;
    const long long x_bytes = ((SP_COLS - 1) * ldb + n_in) * 4;
    const long long y_bytes = ((SP_COLS - 1) * ldd + n_out) * 4;
    const long long a_bytes = (long long)A.nd * A.stride * 4;
    const int nchunks = trans ? A.n_chunks_t : A.n_chunks_n;
    return A.rf == 1 && n_in >= 4 && nchunks <= SP_MAX_CHUNKS && x_bytes < (long long)OOB_OFFSET &&
           y_bytes < (long long)OOB_OFFSET && a_bytes < (long long)OOB_OFFSET;
}

#endif  // part 4

// Everything a launch of the tiled SpMM kernel needs; the launch itself lives in the unit that
// instantiates the kernel for the table's longest chunk.
struct SpLaunch {
    const Chunk *chunks;
    int nchunks;
    const float *vals;
    int stride, ashift;
    const float *B;
    long long ldb;
    float *dst;
    long long ldd;
    int n_out, n_in, batch;
    float alpha, beta;
    int col_tiles, col_group;
    unsigned a_bytes;
    int s_min, s_max;
    int period_tiles;           // window tables: tiles between window rows (0: no renumbering of the row tiles)
    int slot_step;              // table positions between neighbouring diagonals of a chunk, if common (else 0)
    SpEpilogue ep;
    dim3 grid;
    hipStream_t stream;
    int lck;
    bool mixed;                 // some chunk of the table is shorter than lck
};
// The walking kernel's launch (its unit instantiates the kernel); returns hipErrorNotSupported when no
// instantiation fits the table.
struct WalkLaunch {
    const int *tab;
    int ngroups, period, s0, astep4, lck, k, seg_tiles;
    const float *vals, *B;
    long long ldb;
    float *dst;
    long long ldd;
    int n_out, n_in, batch;
    float alpha, beta;
    int col_tiles;
    unsigned a_bytes;
    hipStream_t stream;
    SpEpilogue ep;              // bias, sigmoid and sample at the tiles' exit
};
hipError_t spmm_walk_launch(const WalkLaunch &L);
// The window-table projection's launch (its unit instantiates the kernel for every chunk length and alignment).
struct DwLaunch {
    const int *tab;
    int ngroups, k, period, s0, astep, lck;
    float *vals;
    const float *A;
    long long lda;
    const float *B;
    long long ldb;
    int h, w, batch;
    float alpha, beta;
    unsigned a_bytes, b_bytes, c_bytes;
    int txn, tyn, ndb;
    int subs;                   // batch ranges per workgroup: 1, 2 or 4
    hipStream_t stream;
};
hipError_t dd2dia_window_launch(const DwLaunch &L);
hipError_t dd2dia_window_long_launch(const DwLaunch &L);      // (rows of 9 to 13 diagonals; a unit of its own)
hipError_t spmm_tiled_launch_1_5(const SpLaunch &L);
hipError_t spmm_tiled_launch_6_9(const SpLaunch &L);
hipError_t spmm_tiled_launch_10_13(const SpLaunch &L);

// 8 rows per wave (8 waves per workgroup) keeps four waves on every SIMD
// at the sizes this path is measured on.
#define CUVDIA_SPMM_ARGS L.chunks, L.nchunks, L.vals, L.stride, L.ashift, L.B, L.ldb, L.dst, L.ldd, L.n_out, L.n_in, \
                         L.batch, L.alpha, L.beta, L.col_tiles, L.col_group, L.a_bytes, L.s_min, L.s_max, L.period_tiles, L.slot_step, L.ep
#define CUVDIA_SPMM_LAUNCH_ONE(K, NTAB, EP, MIXED)                                                                    \
    hipLaunchKernelGGL((spmm_tiled_kernel<K, 8, NTAB, EP, MIXED>), L.grid, dim3(512), 0, L.stream, CUVDIA_SPMM_ARGS)
#define CUVDIA_SPMM_LAUNCH_TAB(K, NTAB)                                                                               \
    do {                                                                                                              \
        if (K > 1 && L.mixed) {                                                                                       \
            if (fused) CUVDIA_SPMM_LAUNCH_ONE(K, NTAB, true, (K > 1));                                                \
            else CUVDIA_SPMM_LAUNCH_ONE(K, NTAB, false, (K > 1));                                                     \
        } else {                                                                                                      \
            if (fused) CUVDIA_SPMM_LAUNCH_ONE(K, NTAB, true, false);                                                  \
            else CUVDIA_SPMM_LAUNCH_ONE(K, NTAB, false, false);                                                       \
        }                                                                                                             \
    } while (0)
#define CUVDIA_SPMM_LAUNCH(K)                                                                                         \
    case K:                                                                                                           \
        note_kernel("spmm_tiled_kernel<%d, 8, %d, %s, %s>", K, L.nchunks <= 64 ? 1 : 4, fused ? "true" : "false",     \
                    (K > 1 && L.mixed) ? "true" : "false");                                                           \
        if (L.nchunks <= 64) CUVDIA_SPMM_LAUNCH_TAB(K, 1);                                                            \
        else CUVDIA_SPMM_LAUNCH_TAB(K, 4);                                                                            \
        break;
#if CUVDIA_IN_PART(5)
// rows per wave of the instantiation that serves a window of k rows of lck diagonals whose first shift is
// s0 (0: none).  Instantiated: the centred 3x3, 5x5 and 7x7 windows.  (A 13x13 window needs 13 sets of running
// sums: with the registers that leaves, two waves per SIMD, it ran slower than the tile-by-tile kernel.)
static int walk_rows_per_wave(int lck, int k, int s0)
{
    const int sh = ((s0 % 4) + 4) % 4;
    if (lck == 7 && k == 7 && sh == 1) return 8;
    if (lck == 5 && k == 5 && sh == 2) return 8;
    if (lck == 3 && k == 3 && sh == 3) return 8;
    return 0;
}
int spmm_walk_tile_rows(int lck, int k, int s0) { return 8 * walk_rows_per_wave(lck, k, s0); }
// Tiles per segment of a walking launch, 0 when the walking kernel does not run: no instantiation for the
// window, row counts that its tiles do not divide, or -- unless `forced` -- a launch that would not fill the chip.
// Segments are as long as they can be while the launch still has SP_WALK_WGS workgroups, but no shorter than
// the window has rows: a segment of S tiles stages S + k - 1 blocks.
int spmm_walk_plan(int lck, int k, int s0, int period, long long n_out, long long n_in, long long col_tiles,
                   bool forced, long long *workgroups)
{
    if (workgroups) *workgroups = 0;
    const int rows = spmm_walk_tile_rows(lck, k, s0);
    if (rows == 0 || n_out % rows != 0 || n_in % 4 != 0 || period % rows != 0) return 0;
    const long long tp = period / rows;
    const long long walk_len = (n_out / rows + tp - 1) / tp;
    const long long walks = tp * col_tiles;
    long long nseg = (SP_WALK_WGS + walks - 1) / walks;
    if (nseg > walk_len / k) nseg = walk_len / k;
    if (forced && nseg < 1) nseg = 1;
    if (nseg < 1 || !(forced || nseg * walks >= SP_WALK_MIN_WGS)) return 0;
    const long long seg_tiles = (walk_len + nseg - 1) / nseg;
    if (workgroups) *workgroups = ((walk_len + seg_tiles - 1) / seg_tiles) * walks;
    return (int)seg_tiles;
}
hipError_t spmm_walk_launch(const WalkLaunch &L)
{
    const int rows = spmm_walk_tile_rows(L.lck, L.k, L.s0);
    if (rows == 0) return hipErrorNotSupported;
    if (L.n_out % rows != 0 || L.n_in % 4 != 0 || L.period % rows != 0 || L.seg_tiles < 1) return hipErrorNotSupported;
    const int tp = L.period / rows;
    const int walk_len = (L.n_out / rows + tp - 1) / tp;
    const int nseg = (walk_len + L.seg_tiles - 1) / L.seg_tiles;
    const dim3 grid((unsigned)((long long)nseg * tp * L.col_tiles));
#define CUVDIA_WALK_ARGS L.tab, L.ngroups, L.period, L.s0, L.astep4, L.seg_tiles, L.vals, L.B, L.ldb, L.dst, L.ldd, \
                         L.n_out, L.n_in, L.batch, L.alpha, L.beta, L.col_tiles, L.a_bytes, L.ep
    const bool fused = L.ep.bias != nullptr || L.ep.act != 0;
    note_kernel("spmm_walk_kernel<%d, %d, 8, %d, %s>", L.lck, L.lck, L.lck == 7 ? 1 : L.lck == 5 ? 2 : 3, fused ? "true" : "false");
#define CUVDIA_WALK_LAUNCH(LCK, SH)                                                                                    \
    do {                                                                                                               \
        if (fused) hipLaunchKernelGGL((spmm_walk_kernel<LCK, LCK, 8, SH, true>), grid, dim3(512), 0, L.stream, CUVDIA_WALK_ARGS); \
        else hipLaunchKernelGGL((spmm_walk_kernel<LCK, LCK, 8, SH, false>), grid, dim3(512), 0, L.stream, CUVDIA_WALK_ARGS); \
    } while (0)
    if (L.lck == 7) CUVDIA_WALK_LAUNCH(7, 1);
    else if (L.lck == 5) CUVDIA_WALK_LAUNCH(5, 2);
    else CUVDIA_WALK_LAUNCH(3, 3);
#undef CUVDIA_WALK_LAUNCH
#undef CUVDIA_WALK_ARGS
    return hipGetLastError();
}
#endif
#if CUVDIA_IN_PART(6)
hipError_t dd2dia_window_launch(const DwLaunch &L)
{
    const long long blocks = (long long)L.ngroups * L.ndb * L.tyn * L.txn;
    if (blocks <= 0 || blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    const dim3 grid((unsigned)blocks);
    const int sh = ((L.s0 % 4) + 4) % 4;
#define CUVDIA_DW_ARGS L.tab, L.ngroups, L.k, L.period, L.s0, L.astep, L.vals, L.A, L.lda, L.B, L.ldb, L.h, L.w, L.batch, \
                       L.alpha, L.beta, L.a_bytes, L.b_bytes, L.c_bytes, L.txn, L.tyn, L.ndb
#define CUVDIA_DW_LAUNCH_SUBS(LC, SUBS)                                                                               \
    do {                                                                                                              \
        if (sh == 0) hipLaunchKernelGGL((dd2dia_window_kernel<LC, 0, SUBS>), grid, dim3(256 * SUBS), 0, L.stream, CUVDIA_DW_ARGS); \
        else if (sh == 1) hipLaunchKernelGGL((dd2dia_window_kernel<LC, 1, SUBS>), grid, dim3(256 * SUBS), 0, L.stream, CUVDIA_DW_ARGS); \
        else if (sh == 2) hipLaunchKernelGGL((dd2dia_window_kernel<LC, 2, SUBS>), grid, dim3(256 * SUBS), 0, L.stream, CUVDIA_DW_ARGS); \
        else hipLaunchKernelGGL((dd2dia_window_kernel<LC, 3, SUBS>), grid, dim3(256 * SUBS), 0, L.stream, CUVDIA_DW_ARGS); \
    } while (0)
#define CUVDIA_DW_LAUNCH(LC)                                                                                          \
    case LC:                                                                                                          \
        if (L.subs == 4) CUVDIA_DW_LAUNCH_SUBS(LC, 4);                                                                \
        else if (L.subs == 2) CUVDIA_DW_LAUNCH_SUBS(LC, 2);                                                           \
        else CUVDIA_DW_LAUNCH_SUBS(LC, 1);                                                                            \
        break;
    if (L.lck > CHUNK_MAX) return L.subs == 1 ? dd2dia_window_long_launch(L) : hipErrorNotSupported;
    note_kernel("dd2dia_window_kernel<%d, %d, %d>", L.lck, sh, L.subs);
    switch (L.lck) {
        CUVDIA_DW_LAUNCH(2) CUVDIA_DW_LAUNCH(3) CUVDIA_DW_LAUNCH(4) CUVDIA_DW_LAUNCH(5)
        CUVDIA_DW_LAUNCH(6) CUVDIA_DW_LAUNCH(7) CUVDIA_DW_LAUNCH(8)
        default: return hipErrorNotSupported;
    }
#undef CUVDIA_DW_LAUNCH
#undef CUVDIA_DW_LAUNCH_SUBS
#undef CUVDIA_DW_ARGS
    return hipGetLastError();
}
#endif
#if CUVDIA_IN_PART(7)
hipError_t dd2dia_window_long_launch(const DwLaunch &L)
{
    const long long blocks = (long long)L.ngroups * L.ndb * L.tyn * L.txn;
    if (blocks <= 0 || blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    const dim3 grid((unsigned)blocks);
    const int sh = ((L.s0 % 4) + 4) % 4;
    const int nw = dw_long_rows(L.k, L.lck, L.s0);
#define CUVDIA_DWL_ARGS L.tab, L.ngroups, L.k, L.period, L.s0, L.astep, L.vals, L.A, L.lda, L.B, L.ldb, L.h, L.w, L.batch, \
                        L.alpha, L.beta, L.a_bytes, L.b_bytes, L.c_bytes, L.txn, L.tyn, L.ndb
#define CUVDIA_DWL_LAUNCH_NW(LC, SH)                                                                                   \
    do {                                                                                                               \
        if (nw == 5) hipLaunchKernelGGL((dd2dia_window_long_kernel<LC, SH, 5>), grid, dim3(320), 0, L.stream, CUVDIA_DWL_ARGS); \
        else hipLaunchKernelGGL((dd2dia_window_long_kernel<LC, SH, 7>), grid, dim3(448), 0, L.stream, CUVDIA_DWL_ARGS); \
    } while (0)
#define CUVDIA_DWL_LAUNCH(LC)                                                                                          \
    case LC:                                                                                                           \
        if (sh == 0) CUVDIA_DWL_LAUNCH_NW(LC, 0);                                                                      \
        else if (sh == 1) CUVDIA_DWL_LAUNCH_NW(LC, 1);                                                                 \
        else if (sh == 2) CUVDIA_DWL_LAUNCH_NW(LC, 2);                                                                 \
        else CUVDIA_DWL_LAUNCH_NW(LC, 3);                                                                              \
        break;
    if (nw != 5 && nw != 7) return hipErrorNotSupported;
    note_kernel("dd2dia_window_long_kernel<%d, %d, %d>", L.lck, sh, nw);
    switch (L.lck) {
        CUVDIA_DWL_LAUNCH(9) CUVDIA_DWL_LAUNCH(10) CUVDIA_DWL_LAUNCH(11) CUVDIA_DWL_LAUNCH(12) CUVDIA_DWL_LAUNCH(13)
        default: return hipErrorNotSupported;
    }
#undef CUVDIA_DWL_LAUNCH
#undef CUVDIA_DWL_LAUNCH_NW
#undef CUVDIA_DWL_ARGS
    return hipGetLastError();
}
#endif
#if CUVDIA_IN_PART(1)
hipError_t spmm_tiled_launch_1_5(const SpLaunch &L)
{
    const bool fused = L.ep.bias != nullptr || L.ep.act != 0;
    switch (L.lck) {
        CUVDIA_SPMM_LAUNCH(1) CUVDIA_SPMM_LAUNCH(2) CUVDIA_SPMM_LAUNCH(3) CUVDIA_SPMM_LAUNCH(4) CUVDIA_SPMM_LAUNCH(5)
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}
#endif
#if CUVDIA_IN_PART(2)
hipError_t spmm_tiled_launch_6_9(const SpLaunch &L)
{
    const bool fused = L.ep.bias != nullptr || L.ep.act != 0;
    switch (L.lck) {
        CUVDIA_SPMM_LAUNCH(6) CUVDIA_SPMM_LAUNCH(7) CUVDIA_SPMM_LAUNCH(8) CUVDIA_SPMM_LAUNCH(9)
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}
#endif
#if CUVDIA_IN_PART(3)
hipError_t spmm_tiled_launch_10_13(const SpLaunch &L)
{
    const bool fused = L.ep.bias != nullptr || L.ep.act != 0;
    switch (L.lck) {
        CUVDIA_SPMM_LAUNCH(10) CUVDIA_SPMM_LAUNCH(11) CUVDIA_SPMM_LAUNCH(12) CUVDIA_SPMM_LAUNCH(13)
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}
#endif
#undef CUVDIA_SPMM_LAUNCH
#undef CUVDIA_SPMM_LAUNCH_TAB
#undef CUVDIA_SPMM_LAUNCH_ONE
#undef CUVDIA_SPMM_ARGS

#if CUVDIA_IN_PART(4)
hipError_t launch_spmm_tiled(const DiaView &A, const float *vals, const float *B, long long ldb,
                             float *dst, long long ldd, int batch, bool trans,
                             float alpha, float beta, SpEpilogue ep, hipStream_t stream, int walk, bool *walked)
{
    if (walked) *walked = false;
    const int n_out = trans ? A.w : A.h;
    const int n_in = trans ? A.h : A.w;
    const long long row_tiles = (n_out + SP_ROWS - 1) / SP_ROWS;
    const long long col_tiles = (batch + SP_COLS - 1) / SP_COLS;
    if (row_tiles * col_tiles > 0x7fffffffLL) return hipErrorInvalidValue;
    // Up to 4 column tiles form one group (the diagonals are fetched once per group and row tile); wider
    // batches are walked in groups of 2 column tiles, so that the tiles resident in an XCD stay neighbours
    // along the rows and find each other's dense rows in its L2.
    const int col_group = col_tiles <= 4 ? (int)col_tiles : 2;
    const int lck = trans ? A.max_len_t : A.max_len_n;
    // A window table on a product of many tiles: the walking kernel (with the bias, the sigmoid and the sample at
    // its tiles' exit, if asked for).
    const WalkView &wk = trans ? A.walk_t : A.walk_n;
    if (walk >= 0 && wk.tab_dev != nullptr) {
        WalkLaunch W{wk.tab_dev, wk.ngroups, wk.period, wk.s0, wk.astep4, wk.lck, wk.k, 0, vals, B, ldb, dst, ldd,
                     n_out, n_in, batch, alpha, beta, (int)col_tiles, (unsigned)((long long)A.nd * A.stride * 4), stream, ep};
        const int seg_tiles = spmm_walk_plan(wk.lck, wk.k, wk.s0, wk.period, n_out, n_in, col_tiles, walk > 0, nullptr);
        if (seg_tiles > 0) {
            W.seg_tiles = seg_tiles;
            if (walked) *walked = true;
            return spmm_walk_launch(W);
        }
    }
    if (walk > 0) return hipErrorNotSupported;
    const SpLaunch L{trans ? A.chunks_t_dev : A.chunks_n_dev,
                     trans ? A.n_chunks_t : A.n_chunks_n,
                     vals, A.stride, trans ? 1 : 0, B, ldb, dst, ldd, n_out, n_in, batch, alpha, beta,
                     (int)col_tiles, col_group, (unsigned)((long long)A.nd * A.stride * 4),
                     trans ? A.s_min_t : A.s_min_n, trans ? A.s_max_t : A.s_max_n,
                     (wk.tab_dev != nullptr && wk.period % SP_ROWS == 0 && row_tiles * col_tiles > SP_RENUMBER_MIN_TILES)
                         ? wk.period / SP_ROWS : 0,
                     trans ? A.slot_step_t : A.slot_step_n, ep,
                     dim3((unsigned)(row_tiles * col_tiles)), stream, lck,
                     (trans ? A.min_len_t : A.min_len_n) != lck};
    if (lck <= 5) return spmm_tiled_launch_1_5(L);
    if (lck <= 9) return spmm_tiled_launch_6_9(L);
    return spmm_tiled_launch_10_13(L);
}

hipError_t launch_dd2dia_generic(const DiaView &C, float *vals, const float *A, long long lda,
                                 const float *B, long long ldb, int batch,
                                 float alpha, float beta, hipStream_t stream)
{
    const unsigned gx = (unsigned)((C.h + 255) / 256);
    int done = 0;
    while (done < C.nd) {
        const int slab = C.nd - done < 65535 ? C.nd - done : 65535;
        note_kernel("dd2dia_generic_kernel");
        hipLaunchKernelGGL(dd2dia_generic_kernel, dim3(gx, (unsigned)slab), dim3(256), 0, stream,
                           C.offsets_dev + done, vals + (long long)done * C.stride, C.stride,
                           C.h, C.w, C.rf, A, lda, B, ldb, batch, alpha, beta);
        done += slab;
    }
    return hipGetLastError();
}

hipError_t launch_avg_diagonals(const DiaView &A, const float *vals, float *dst, hipStream_t stream)
{
    int done = 0;
    while (done < A.nd) {
        const int slab = A.nd - done < 65535 ? A.nd - done : 65535;
        hipLaunchKernelGGL(avg_diagonals_kernel, dim3((unsigned)slab), dim3(AVG_THREADS), 0, stream,
                           A.offsets_dev + done, vals + (long long)done * A.stride, A.stride, A.h, A.w, dst + done);
        done += slab;
    }
    return hipGetLastError();
}

hipError_t launch_axpby(float *W, const float *dW, long long n, float alpha, float beta, hipStream_t stream)
{
    if (n <= 0) return hipSuccess;
    const unsigned long long wa = reinterpret_cast<unsigned long long>(W), da = reinterpret_cast<unsigned long long>(dW);
    const bool vec = (wa & 15u) == (da & 15u) && (wa & 3u) == 0 && n >= 8;
    const long long head = vec ? (long long)(((16u - (wa & 15u)) & 15u) / 4u) : 0;
    const long long items = vec ? (n - head) / 4 : n;
    long long blocks = (items + AXPBY_THREADS - 1) / AXPBY_THREADS;
    if (blocks > 256 * 16) blocks = 256 * 16;         // 16 workgroups per CU, grid-stride beyond that
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(axpby_kernel, dim3((unsigned)blocks), dim3(AXPBY_THREADS), 0, stream, W, dW, n, alpha, beta,
                       (int)head, (int)vec);
    return hipGetLastError();
}

hipError_t launch_momentum(float *W, float *M, const float *dW, long long n, float lr, float mw, float l2,
                           hipStream_t stream)
{
    if (n <= 0) return hipSuccess;
    const unsigned long long wa = reinterpret_cast<unsigned long long>(W), ma = reinterpret_cast<unsigned long long>(M),
                             da = reinterpret_cast<unsigned long long>(dW);
    const bool vec = (wa & 15u) == (da & 15u) && (wa & 15u) == (ma & 15u) && (wa & 3u) == 0 && n >= 8;
    const long long head = vec ? (long long)(((16u - (wa & 15u)) & 15u) / 4u) : 0;
    const long long items = vec ? (n - head) / 4 : n;
    long long blocks = (items + AXPBY_THREADS - 1) / AXPBY_THREADS;
    if (blocks > 256 * 16) blocks = 256 * 16;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(momentum_kernel, dim3((unsigned)blocks), dim3(AXPBY_THREADS), 0, stream, W, M, dW, n, lr, mw, l2,
                       (int)head, (int)vec);
    return hipGetLastError();
}

bool dd2dia_tiled_ok(const DiaView &C, long long lda, long long ldb, int batch)
{
    // buffer resources address 32-bit byte offsets below the out-of-range marker
    const long long nb = batch > 0 ? batch : 1;
    const long long a_bytes = ((nb - 1) * lda + C.h) * 4;
    const long long b_bytes = ((nb - 1) * ldb + C.w) * 4;
    const long long c_bytes = (long long)C.nd * C.stride * 4;
    return C.rf == 1 && C.max_len_p >= 1 && a_bytes < (long long)OOB_OFFSET &&
           b_bytes < (long long)OOB_OFFSET && c_bytes < (long long)OOB_OFFSET;
}

int dd2dia_slab_columns(const DiaView &C, long long lda, long long ldb)
{
    // ((n - 1) * ld + rows) * 4 < OOB_OFFSET for both operands
    const long long floats = (long long)OOB_OFFSET / 4;
    auto cols = [&](long long ld, long long rows) -> long long {
        if (rows >= floats || ld <= 0) return 0;
        return (floats - rows - 1) / ld + 1;
    };
    const long long n = std::min(cols(lda, C.h), cols(ldb, C.w));
    const long long whole = n / DD2DIA_SLAB_MIN * DD2DIA_SLAB_MIN;
    return whole >= DD2DIA_SLAB_MIN ? (int)std::min<long long>(whole, 1 << 30) : 0;
}

// Workgroups of the window-table projection on these operands, 0 where it does not apply: no window table,
// chunks longer than CHUNK_MAX or shorter than 2, a period, group rows or row counts that are no multiples of 4
// (its 16-byte pieces then straddle the operands' ends).
long long dd2dia_window_workgroups(const DiaView &C, int batch, int *txn, int *tyn, int *ndb)
{
    const WalkView &wk = C.walk_n;
    if (wk.tab_dev == nullptr || wk.lck < 2 || wk.lck > SP_CHUNK_MAX || !wk.rows4 || wk.period % 4 != 0 ||
        C.h % 4 != 0 || C.w % 4 != 0 || batch < 1 || wk.astep4 % 4 != 0)
        return 0;
    const long long image_rows = ((long long)C.h + wk.period - 1) / wk.period;
    const long long tx = ((long long)wk.period + 63) / 64, ty = (image_rows + 3) / 4,
                    db = wk.lck > CHUNK_MAX ? (wk.k + dw_long_rows(wk.k, wk.lck, wk.s0) - 1) / dw_long_rows(wk.k, wk.lck, wk.s0) : (wk.k + 7) / 8;
    const long long total = tx * ty * db * wk.ngroups;
    if (total > 0x7fffffffLL || (long long)4 * ty * wk.period + 64 * tx >= (1LL << 30)) return 0;
    if (txn) *txn = (int)tx;
    if (tyn) *tyn = (int)ty;
    if (ndb) *ndb = (int)db;
    return total;
}

// Batch ranges per workgroup the window-table projection runs with on a launch of so many workgroups (tiles):
// 1 when the tiles alone fill the chip (four workgroups of 4 waves per CU), 2 or 4 when it takes that many ranges
// of the batch per tile to get there.  The smaller the window, the less a tile saves over the chunk-by-chunk
// kernel and the more tiles it takes (measured on 7 x 7, 5 x 5 and 3 x 3 windows of maps 256 to 1024 wide at
// batch 32 to 512: ahead from 768, 1024 and 1536 tiles on, the 3 x 3 only from batch 128).
int dd2dia_window_subs(const DiaView &C, long long workgroups)
{
    const int slots = C.walk_n.k * C.walk_n.lck;
    const long long min_wgs = slots >= 49 ? DW_MIN_WGS : slots >= 25 ? DW_MIN_WGS * 4 / 3 : DW_MIN_WGS * 2;
    if (C.walk_n.lck > CHUNK_MAX) return 1;            // (rows of 9 to 13 diagonals: one range only)
    return workgroups >= min_wgs ? 1 : 2 * workgroups >= min_wgs ? 2 : 4;
}
// Whether the automatic choice takes the window-table projection: enough tiles to fill the chip and a map no
// narrower than a tile's 64 positions (lanes would idle).  With 2 or 4 batch ranges per tile only windows of 49
// slots or more, and two ranges only from batch 512 on: a 7 x 7 window on a 256-wide map (256 tiles, 4 ranges)
// measured 1.2 - 1.5 times the chunk-by-chunk kernel's rate at batch 32 to 2048, on 320- and 384-wide maps (400 and
// 576 tiles, 2 ranges) 1.1 - 1.6 times from batch 512 and 0.86 - 0.98 below; 5 x 5 windows on those maps 0.6 - 1.0.
bool dd2dia_window_by_size(const DiaView &C, int batch, long long workgroups)
{
    const int slots = C.walk_n.k * C.walk_n.lck;
    const long long min_wgs = slots >= 49 ? DW_MIN_WGS : slots >= 25 ? DW_MIN_WGS * 4 / 3 : DW_MIN_WGS * 2;
    const int subs = dd2dia_window_subs(C, workgroups);
    if (C.walk_n.period < 64) return false;
    if (C.walk_n.lck > CHUNK_MAX) {
        // Rows of 9 to 13 diagonals.  Measured on 9 x 9 to 13 x 13 windows, 1 to 4 channels, maps 128 to 1024 wide,
        // batch 16 to 1024: 1.08 - 1.5 times the chunk-by-chunk kernel's rate where taken, 0.75 - 1.0 where not
        // (windows of 11 rows -- 11 of 14 wave slots -- of one channel, maps 128 wide).
        const int nw = dw_long_rows(C.walk_n.k, C.walk_n.lck, C.walk_n.s0), blocks = (C.walk_n.k + nw - 1) / nw;
        const bool full = C.walk_n.k * 10 >= blocks * nw * 9;      // at most a tenth of the wave slots idle
        const int units = C.walk_n.k * C.walk_n.ngroups;
        if (C.walk_n.period < 192) return false;
        if (workgroups >= 4096) return true;
        if (full) return workgroups >= 1024 || (workgroups >= 512 && C.walk_n.period >= 256);
        return units >= 22 && workgroups >= 1024;
    }
    if (subs * workgroups < min_wgs) return false;
    if (subs == 1) return slots >= 25 || batch >= 128;
    return slots >= 49 && batch >= (subs == 2 ? 512 : 32);
}

hipError_t launch_dd2dia_tiled(const DiaView &C, float *vals, const float *A, long long lda,
                               const float *B, long long ldb, int batch,
                               float alpha, float beta, hipStream_t stream, int window, bool *windowed)
{
    if (windowed) *windowed = false;
    if (window >= 0) {
        int txn = 0, tyn = 0, ndb = 0;
        long long wgs = dd2dia_window_workgroups(C, batch, &txn, &tyn, &ndb);
        // (a lane's byte offsets run up to 16 columns past the batch and must stay below 2^32)
        if (((long long)batch + 16) * std::max(lda, ldb) * 4 >= (1LL << 32)) wgs = 0;
        if (wgs > 0 && (window > 0 || dd2dia_window_by_size(C, batch, wgs))) {
            const WalkView &wk = C.walk_n;
            const DwLaunch L{wk.tab_dev, wk.ngroups, wk.k, wk.period, wk.s0, wk.astep4 / 4, wk.lck, vals, A, lda, B, ldb,
                             C.h, C.w, batch, alpha, beta,
                             (unsigned)((((long long)batch - 1) * lda + C.h) * 4),
                             (unsigned)((((long long)batch - 1) * ldb + C.w) * 4),
                             (unsigned)((long long)C.nd * C.stride * 4), txn, tyn, ndb,
                             dd2dia_window_subs(C, wgs), stream};
            if (windowed) *windowed = true;
            return dd2dia_window_launch(L);
        }
    }
    if (window > 0) return hipErrorNotSupported;
    // 16-byte loads of A need an aligned base and leading dimension and whole
    // groups of 4 rows; row tiles start at multiples of 256 and lanes at
    // multiples of 4 rows.
    const bool a_vec = (reinterpret_cast<unsigned long long>(A) % 16 == 0) && (lda % 4 == 0) && (C.h % 4 == 0);
    const unsigned a_bytes = batch > 0 ? (unsigned)((((long long)batch - 1) * lda + C.h) * 4) : 0u;
    const unsigned b_bytes = batch > 0 ? (unsigned)((((long long)batch - 1) * ldb + C.w) * 4) : 0u;
    const unsigned c_bytes = (unsigned)((long long)C.nd * C.stride * 4);
    // without pairs the units are the chunks themselves, in table order
    // (pairs only with 16-byte loads of A: the dword-load variant of the pair
    // body needs more registers than a wave has)
    const bool use_units = C.n_units < C.n_chunks_p && a_vec;
    // A table with runs longer than CHUNK_MAX is walked in the long chunks of
    // the products' table instead (a 13-wide window row as one unit rather
    // than two that cannot pair): the same registers as a pair, half the
    // loads and LDS traffic per FMA.  (16-byte loads of A only, as for pairs.)
    const bool long_chunks = C.max_len_n > CHUNK_MAX && a_vec;
    // A table with a pair further apart than one band holds runs the form that shares B's rows instead of A's
    // (DD_SHIFTED) -- if its chunks have at least 4 shifts: pairs of shorter ones measured slower than the chunks on
    // their own (3 x 3 windows on a 512-wide map: 409 against 310 us at batch 512), so those stay single.  Pairs that
    // fit a band keep the forms that share A's rows: the band forms run a 7 x 7 window on a 128-wide map at batch
    // 2048 in 81 us, the shifted form in 145.
    const bool far = use_units && !long_chunks && C.pair_delta_max > PAIR_BAND_DELTA;
    const bool shifted = far && C.max_len_p >= 4;
    const bool pairs = use_units && !long_chunks && (!far || shifted);
    const bool wide = pairs && !shifted && C.pair_delta_max > PAIR_NARROW_DELTA;      // some pair needs the 520-row band
    const Unit *units = pairs ? C.units_dev : C.single_units_dev;      // the single units count 0, 1, 2, ...
    const int nunits = long_chunks ? C.n_chunks_n : pairs ? C.n_units : C.n_chunks_p;
    const Chunk *table = long_chunks ? C.chunks_n_dev : C.chunks_p_dev;
    const int lc = long_chunks ? C.max_len_n : C.max_len_p;
    const int tile_rows = (pairs && !shifted) ? DD_ROWS : lc > CHUNK_MAX ? dd_short_rows<SP_CHUNK_MAX>() : dd_short_rows<CHUNK_MAX>();
    const long long row_tiles = ((long long)C.h + (shifted ? C.pair_delta_max : 0) + tile_rows - 1) / tile_rows;
    const int ub = DdBlock::units(nunits), rb = DdBlock::rows(nunits);
    const int blocked = row_tiles * nunits > DD_BLOCKED_MIN_TILES ? 1 : 0;
    const long long blocks = blocked ? ((row_tiles + rb - 1) / rb) * ((nunits + ub - 1) / ub) * (long long)(rb * ub)
                                     : row_tiles * nunits;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    const dim3 grid((unsigned)blocks);
#define CUVDIA_DD_ARGS table, units, nunits, vals, C.stride, A, lda, B, ldb, C.h, C.w, batch, alpha, beta, \
                       a_bytes, b_bytes, c_bytes, blocked, (int)row_tiles
#define CUVDIA_DD_LAUNCH(L)                                                                              \
    case L:                                                                                              \
        if (shifted) {                                                                                   \
            hipLaunchKernelGGL((dd2dia_tiled_kernel<L, true, true, DD_SHIFTED>), grid, dim3(256), 0, stream, CUVDIA_DD_ARGS);  \
        } else if (wide) {                                                                               \
            hipLaunchKernelGGL((dd2dia_tiled_kernel<L, true, true, DD_WIDE>), grid, dim3(512), 0, stream, CUVDIA_DD_ARGS);  \
        } else if (pairs) {                                                                              \
            hipLaunchKernelGGL((dd2dia_tiled_kernel<L, true, true>), grid, dim3(512), 0, stream, CUVDIA_DD_ARGS);  \
        } else {                                                                                         \
            if (a_vec) hipLaunchKernelGGL((dd2dia_tiled_kernel<L, true, false>), grid, dim3(256), 0, stream, CUVDIA_DD_ARGS);  \
            else hipLaunchKernelGGL((dd2dia_tiled_kernel<L, false, false>), grid, dim3(256), 0, stream, CUVDIA_DD_ARGS);       \
        }                                                                                                \
        break;
#define CUVDIA_DD_LAUNCH_LONG(L)                                                                         \
    case L:                                                                                              \
        hipLaunchKernelGGL((dd2dia_tiled_kernel<L, true, false>), grid, dim3(256), 0, stream, CUVDIA_DD_ARGS);      \
        break;
    if (lc > CHUNK_MAX) note_kernel("dd2dia_tiled_kernel<%d, true, false, 0>", lc);
    else note_kernel("dd2dia_tiled_kernel<%d, %s, %s, %d>", lc, (shifted || wide || pairs || a_vec) ? "true" : "false",
                     (shifted || wide || pairs) ? "true" : "false", shifted ? DD_SHIFTED : wide ? DD_WIDE : DD_NARROW);
    switch (lc) {
        CUVDIA_DD_LAUNCH(1) CUVDIA_DD_LAUNCH(2) CUVDIA_DD_LAUNCH(3) CUVDIA_DD_LAUNCH(4)
        CUVDIA_DD_LAUNCH(5) CUVDIA_DD_LAUNCH(6) CUVDIA_DD_LAUNCH(7) CUVDIA_DD_LAUNCH(8)
        CUVDIA_DD_LAUNCH_LONG(9) CUVDIA_DD_LAUNCH_LONG(10) CUVDIA_DD_LAUNCH_LONG(11) CUVDIA_DD_LAUNCH_LONG(12)
        CUVDIA_DD_LAUNCH_LONG(13)
        default: return hipErrorInvalidValue;
    }
#undef CUVDIA_DD_LAUNCH_LONG
#undef CUVDIA_DD_LAUNCH
#undef CUVDIA_DD_ARGS
    return hipGetLastError();
}

// ------------------------------------------------- tables without allocation --
//
// The table block of the allocation-free entry point: the device copy of the
// offset table and of one chunk table, which a descriptor keeps in memory it
// allocates.  Every GPU holds its own copy of the array at its own address;
// the name below is only the host-side handle that hipGetSymbolAddress turns
// into that address, once per device.
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];
static_assert(NOALLOC_MAX_CHUNKS >= SP_MAX_CHUNKS, "every table the tiled product accepts fits the static array");

// One launch carries up to NOALLOC_PIECE_BYTES of table in its kernel
// arguments (copied by the runtime when the launch is enqueued or captured,
// so the host buffer may go away at once and nothing is staged or allocated).
struct NoallocPiece {
    unsigned w[NOALLOC_PIECE_BYTES / 4];
};
__global__ __launch_bounds__(256) void noalloc_fill_kernel(NoallocPiece piece, unsigned *dst, int nwords)
{
    for (int i = threadIdx.x; i < nwords; i += 256) dst[i] = piece.w[i];
}

hipError_t noalloc_scratch(unsigned char **out)
{
    constexpr int MAX_DEVICES = 64;
    static std::mutex mutex;
    static unsigned char *ptrs[MAX_DEVICES] = {};
    *out = nullptr;
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return e;
    if (device < 0 || device >= MAX_DEVICES) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mutex);
    if (!ptrs[device]) {
        unsigned char *p = nullptr;
        e = hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        ptrs[device] = p;
    }
    *out = ptrs[device];
    return hipSuccess;
}

hipError_t noalloc_upload(unsigned char *dst_dev, const void *src_host, size_t bytes, hipStream_t stream)
{
    const unsigned char *src = static_cast<const unsigned char *>(src_host);
    for (size_t at = 0; at < bytes; at += NOALLOC_PIECE_BYTES) {
        const size_t n = bytes - at < NOALLOC_PIECE_BYTES ? bytes - at : NOALLOC_PIECE_BYTES;
        NoallocPiece piece{};
        std::memcpy(piece.w, src + at, n);
        hipLaunchKernelGGL(noalloc_fill_kernel, dim3(1), dim3(256), 0, stream, piece,
                           reinterpret_cast<unsigned *>(dst_dev + at), (int)((n + 3) / 4));
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

#endif  // part 4

}  // namespace cuvdia
