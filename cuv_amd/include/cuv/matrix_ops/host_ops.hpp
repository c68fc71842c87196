// host_memory_space twins of the DIA operations.
//
// The reference compiles every operation of this path for both memory spaces
// (src/cuv/matrix_ops/spmv.cu:145-220,248-253,
// src/cuv/matrix_ops/densedense_to_sparse.cu:204-252,310-319,
// src/cuv/matrix_ops/diagonals.cu:24-51), and code written against it calls
// prod / spmv / densedense_to_dia on host matrices too.  These are plain
// single-threaded loops in the reference's element order, header-only, with
// no dependency beyond the container headers: the device overloads in
// matrix_ops.hpp, densedense_to_sparse.hpp and diagonals.hpp are the product,
// these keep host-side callers compiling and give them the same numbers the
// reference's host path gives (for densedense_to_dia: the numbers of its
// documented contract, see below).
#ifndef __CUV_DIA_HOST_OPS_HPP__
#define __CUV_DIA_HOST_OPS_HPP__

#include <algorithm>
#include <vector>

#include <cuv/basics/dia_matrix.hpp>
#include <cuv/basics/tensor.hpp>
#include <cuv/matrix_ops/densedense_to_sparse.hpp>

namespace cuv {
namespace detail {

// One column: y = factC*y + factAv*op(A)*x, walking the table diagonal by
// diagonal (src/cuv/matrix_ops/spmv.cu:145-200).  factC == 0 overwrites y
// without reading it (:152-156).  A diagonal lying outside the matrix
// contributes nothing (the reference's unsigned arithmetic wraps there).
inline void host_dia_column(const dia_matrix<float, host_memory_space> &A, const float *x, float *y, char transA,
                            float factAv, float factC)
{
    const long long h = A.h(), w = A.w(), rf = A.row_fact(), stride = A.stride();
    const long long n_out = transA == 't' ? w : h;
    if (factC == 0.f) std::fill(y, y + n_out, 0.f);
    else for (long long i = 0; i < n_out; ++i) y[i] = y[i] * factC;
    const std::vector<int> &offsets = A.host_offsets();
    const float *vals = A.vec().ptr();
    for (int d = 0; d < A.num_dia(); ++d) {
        const long long k = offsets[d];
        const float *diag = vals + (long long)d * stride;
        if (transA == 't') {
            const long long out0 = std::max(0LL, k), in0 = rf * std::max(0LL, -k);
            const long long count = std::min((h - in0) / rf, w - out0);
            for (long long n = 0; n < count; ++n)
                for (long long q = 0; q < rf; ++q) {
                    const long long r = in0 + n * rf + q;
                    y[out0 + n] += factAv * diag[r] * x[r];
                }
        } else {
            const long long out0 = rf * std::max(0LL, -k), in0 = std::max(0LL, k);
            const long long count = std::min(h - out0, rf * (w - in0));
            for (long long n = 0; n < count; ++n) y[out0 + n] += factAv * diag[out0 + n] * x[in0 + n / rf];
        }
    }
}

}  // namespace detail

/// dst = factC*dst + factAv*op(A)*v on the host (src/cuv/matrix_ops/spmv.cu:145-200).
inline void spmv(tensor<float, host_memory_space> &dst, const dia_matrix<float, host_memory_space> &A,
                 const tensor<float, host_memory_space> &v, char transA = 'n',
                 const float &factAv = 1.f, const float &factC = 0.f)
{
    cuvAssert(transA == 'n' || transA == 't');
    if (transA == 't') {
        cuvAssert(A.h() == v.size());
        cuvAssert(A.w() == dst.size());
    } else {
        cuvAssert(A.w() == v.size());
        cuvAssert(A.h() == dst.size());
    }
    detail::host_dia_column(A, v.ptr(), dst.ptr(), transA, factAv, factC);
}

/// dst = factC*dst + factAB*op(A)*B on the host, one spmv per column
/// (src/cuv/matrix_ops/spmv.cu:203-220).
inline void prod(tensor<float, host_memory_space, column_major> &dst, const dia_matrix<float, host_memory_space> &A,
                 const tensor<float, host_memory_space, column_major> &B, char transA = 'n', char transB = 'n',
                 const float &factAB = 1.f, const float &factC = 0.f)
{
    cuvAssert(dst.shape().size() == 2);
    cuvAssert(B.shape().size() == 2);
    cuvAssert(transB == 'n');
    cuvAssert(transA == 'n' || transA == 't');
    cuvAssert(dst.shape()[1] == B.shape()[1]);
    if (transA == 't') {
        cuvAssert(A.h() == B.shape()[0]);
        cuvAssert(A.w() == dst.shape()[0]);
    } else {
        cuvAssert(A.w() == B.shape()[0]);
        cuvAssert(A.h() == dst.shape()[0]);
    }
    const size_t n_in = B.shape()[0], n_out = dst.shape()[0];
    for (size_t c = 0; c < B.shape()[1]; ++c)
        detail::host_dia_column(A, B.ptr() + c * n_in, dst.ptr() + c * n_out, transA, factAB, factC);
}

/// C = factC*C + factAB*proj(A*B') on C's stored diagonals, on the host: the
/// contract documented in src/cuv/matrix_ops/densedense_to_sparse.hpp:107-121,
/// summed in the order of the reference's host loop
/// (densedense_to_sparse.cu:204-252: batch column by batch column for every
/// slot).  That loop itself adds into C and never reads the two factors; with
/// the defaults on a zeroed C -- all the reference's own tests use -- the two
/// agree.  factC == 0 never reads C.
inline void densedense_to_dia(dia_matrix<float, host_memory_space> &C, const host_block_descriptor<float> &,
                              const tensor<float, host_memory_space, column_major> &A,
                              const tensor<float, host_memory_space, column_major> &B,
                              const float &factAB = 1.f, const float &factC = 0.f)
{
    cuvAssert(A.shape().size() == 2);
    cuvAssert(B.shape().size() == 2);
    cuvAssert(C.w() == B.shape()[0]);
    cuvAssert(C.h() == A.shape()[0]);
    cuvAssert(A.shape()[1] == B.shape()[1]);
    const long long h = C.h(), w = C.w(), rf = C.row_fact(), stride = C.stride(), batch = A.shape()[1];
    const std::vector<int> &offsets = C.host_offsets();
    std::vector<float> sum((size_t)std::max(h, 1LL));
    for (int d = 0; d < C.num_dia(); ++d) {
        const long long k = offsets[d];
        const long long row0 = rf * std::max(0LL, -k), col0 = std::max(0LL, k);
        const long long count = std::min(h - row0, rf * (w - col0));
        if (count <= 0) continue;
        std::fill(sum.begin(), sum.begin() + count, 0.f);
        for (long long c = 0; c < batch; ++c) {
            const float *a = A.ptr() + c * h + row0;
            const float *b = B.ptr() + c * w + col0;
            for (long long n = 0; n < count; ++n) sum[n] += a[n] * b[n / rf];
        }
        float *dst = C.vec().ptr() + (long long)d * stride + row0;
        if (factC == 0.f) for (long long n = 0; n < count; ++n) dst[n] = factAB * sum[n];
        else for (long long n = 0; n < count; ++n) dst[n] = factC * dst[n] + factAB * sum[n];
    }
}

/// dst[d] = mean of stored diagonal d over its valid slots, on the host
/// (src/cuv/matrix_ops/diagonals.cu:24-51).  A diagonal without valid slots yields 0.
inline void avg_diagonals(tensor<float, host_memory_space> &dst, const dia_matrix<float, host_memory_space> &dia)
{
    cuvAssert(dia.row_fact() == 1);
    cuvAssert((size_t)dia.num_dia() == (size_t)dst.size());
    const long long h = dia.h(), w = dia.w(), stride = dia.stride();
    const std::vector<int> &offsets = dia.host_offsets();
    for (int d = 0; d < dia.num_dia(); ++d) {
        const long long k = offsets[d];
        const long long row0 = std::max(0LL, -k), col0 = std::max(0LL, k);
        const long long count = std::min(h - row0, w - col0);
        const float *x = dia.vec().ptr() + (long long)d * stride + row0;
        float s = 0.f;
        for (long long n = 0; n < count; ++n) s += x[n];
        dst.ptr()[d] = count > 0 ? s / (float)count : 0.f;
    }
}

}  // namespace cuv
#endif
