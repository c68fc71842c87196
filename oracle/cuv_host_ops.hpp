// host_memory_space operations backed by the C oracle, for tests only.
//
// TEST INFRASTRUCTURE: these functions give C++ tests the reference's
// "run the host path and the device path on the same inputs" pattern
// (src/tests/spmv.cpp:103-143, src/tests/densedense_to_dia.cpp:166-197).  They
// forward to the C oracle (dia_oracle.h), which restates the reference's host
// loops, and live in namespace cuv_oracle so that a test says which side of a
// comparison is the checker: cuv_oracle::prod is the oracle, cuv::prod on host
// operands is the product's own host twin (cuv/matrix_ops/host_ops.hpp).  The
// product headers under cuv_amd/include never include this file.
#ifndef CUV_HOST_OPS_ORACLE_HPP
#define CUV_HOST_OPS_ORACLE_HPP

#include <cuv/basics/dia_matrix.hpp>
#include <cuv/basics/tensor.hpp>
#include <cuv/matrix_ops/densedense_to_sparse.hpp>

#include "dia_oracle.h"

namespace cuv_oracle {
using namespace cuv;

// src/cuv/matrix_ops/spmv.cu:145-200 (asserts :159-160, :180-181)
inline void spmv(tensor<float, host_memory_space> &dst, const dia_matrix<float, host_memory_space> &A,
                 const tensor<float, host_memory_space> &v, char transA = 'n',
                 const float &factAv = 1.f, const float &factC = 0.f)
{
    if (transA == 't') {
        cuvAssert(A.h() == v.size());
        cuvAssert(A.w() == dst.size());
    } else {
        cuvAssert(A.w() == v.size());
        cuvAssert(A.h() == dst.size());
    }
    const int rc = oracle_spmv_f32((int)A.h(), (int)A.w(), A.num_dia(), (int)A.stride(), A.row_fact(),
                                   A.host_offsets().data(), A.vec().ptr(), v.ptr(), dst.ptr(), transA, factAv, factC);
    cuvAssert(rc == 0);
}

// src/cuv/matrix_ops/spmv.cu:203-220
inline void prod(tensor<float, host_memory_space, column_major> &dst, const dia_matrix<float, host_memory_space> &A,
                 const tensor<float, host_memory_space, column_major> &B, char transA = 'n', char transB = 'n',
                 const float &factAB = 1.f, const float &factC = 0.f)
{
    cuvAssert(dst.shape().size() == 2);
    cuvAssert(B.shape().size() == 2);
    cuvAssert(transB == 'n');
    cuvAssert(dst.shape()[1] == B.shape()[1]);
    if (transA == 't') {
        cuvAssert(A.h() == B.shape()[0]);
        cuvAssert(A.w() == dst.shape()[0]);
    } else {
        cuvAssert(A.w() == B.shape()[0]);
        cuvAssert(A.h() == dst.shape()[0]);
    }
    const int rc = oracle_prod_dia_f32((int)A.h(), (int)A.w(), A.num_dia(), (int)A.stride(), A.row_fact(),
                                       A.host_offsets().data(), A.vec().ptr(), B.ptr(), dst.ptr(),
                                       (int)B.shape()[1], transA, factAB, factC);
    cuvAssert(rc == 0);
}

// Documented contract C = factC*C + factAB*proj(A*B') in the host loop's order
// (src/cuv/matrix_ops/densedense_to_sparse.cu:204-252 never reads the factors;
// with the defaults on a zeroed C, which is all the reference tests use, the
// two coincide).
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
    const int rc = oracle_dd2dia_f32((int)C.h(), (int)C.w(), C.num_dia(), (int)C.stride(), C.row_fact(),
                                     C.host_offsets().data(), C.vec().ptr(), A.ptr(), B.ptr(), (int)A.shape()[1],
                                     factAB, factC);
    cuvAssert(rc == 0);
}

// The host loop exactly as the reference wrote it: C += proj(A*B').
inline void densedense_to_dia_literal(dia_matrix<float, host_memory_space> &C,
                                      const tensor<float, host_memory_space, column_major> &A,
                                      const tensor<float, host_memory_space, column_major> &B)
{
    const int rc = oracle_dd2dia_literal_f32((int)C.h(), (int)C.w(), C.num_dia(), (int)C.stride(), C.row_fact(),
                                             C.host_offsets().data(), C.vec().ptr(), A.ptr(), B.ptr(),
                                             (int)A.shape()[1]);
    cuvAssert(rc == 0);
}

// Mean of every stored diagonal over its valid slots
// (src/cuv/matrix_ops/diagonals.cu:24-51).
inline void avg_diagonals(tensor<float, host_memory_space> &dst, const dia_matrix<float, host_memory_space> &dia)
{
    cuvAssert(dia.row_fact() == 1);
    cuvAssert((size_t)dia.num_dia() == (size_t)dst.size());
    const int rc = oracle_avg_diagonals_f32((int)dia.h(), (int)dia.w(), dia.num_dia(), (int)dia.stride(),
                                            dia.host_offsets().data(), dia.vec().ptr(), dst.ptr());
    cuvAssert(rc == 0);
}

// W = -learnrate*dW + (1 - learnrate*decay)*W, element by element in fp32
// (src/cuv/tensor_ops/rprop.cu:331-346).
template <class L>
inline void learn_step_weight_decay(tensor<float, host_memory_space, L> &W, const tensor<float, host_memory_space, L> &dW,
                                    const float &learnrate, const float &decay = 0.0f, const float &sparsedecay = 0.0f)
{
    (void)sparsedecay;
    cuvAssert(dW.ptr());
    cuvAssert(W.ptr());
    cuvAssert(W.size() == dW.size());
    const float alpha = -learnrate, beta = 1.f - learnrate * decay;
    float *w = W.ptr();
    const float *d = dW.ptr();
    for (size_t i = 0; i < (size_t)W.size(); ++i) w[i] = alpha * d[i] + beta * w[i];
}

// m = momentum_weight*m - learnrate*(dW + decay*W); W += m, following the device kernel
// (src/cuv/tensor_ops/rprop.cu:158-170), whose decay term shrinks the weights.
template <class L>
inline void learn_step_weight_decay_momentum(tensor<float, host_memory_space, L> &W,
                                             tensor<float, host_memory_space, L> &momentum,
                                             const tensor<float, host_memory_space, L> &dW, const float &learnrate,
                                             const float &momentum_weight = 0.9f, const float &decay = 0.0f,
                                             const float &sparsedecay = 0.0f)
{
    (void)sparsedecay;
    cuvAssert(dW.ptr());
    cuvAssert(W.ptr());
    cuvAssert(W.size() == dW.size());
    cuvAssert(W.size() == momentum.size());
    float *w = W.ptr(), *mo = momentum.ptr();
    const float *d = dW.ptr();
    for (size_t i = 0; i < (size_t)W.size(); ++i) {
        const float m = momentum_weight * mo[i] - learnrate * (d[i] + decay * w[i]);
        w[i] += m;
        mo[i] = m;
    }
}

// Dense C = factC*C + factAB*op(A)*op(B), fp64 accumulation: stands in for the
// CBLAS sgemm the reference cross-checks against (src/cuv/matrix_ops/matrix_ops.cu:177-304).
inline void prod(tensor<float, host_memory_space, column_major> &dst,
                 const tensor<float, host_memory_space, column_major> &A,
                 const tensor<float, host_memory_space, column_major> &B, char transA = 'n', char transB = 'n',
                 const float &factAB = 1.f, const float &factC = 0.f)
{
    const unsigned m = transA == 'n' ? A.shape()[0] : A.shape()[1];
    const unsigned k = transA == 'n' ? A.shape()[1] : A.shape()[0];
    const unsigned kb = transB == 'n' ? B.shape()[0] : B.shape()[1];
    const unsigned n = transB == 'n' ? B.shape()[1] : B.shape()[0];
    cuvAssert(k == kb);
    cuvAssert(dst.shape()[0] == m && dst.shape()[1] == n);
    for (unsigned i = 0; i < m; ++i)
        for (unsigned j = 0; j < n; ++j) {
            double s = 0;
            for (unsigned l = 0; l < k; ++l) {
                const float a = transA == 'n' ? (float)A(i, l) : (float)A(l, i);
                const float b = transB == 'n' ? (float)B(l, j) : (float)B(j, l);
                s += (double)a * b;
            }
            const double old = factC == 0.f ? 0.0 : (double)factC * (float)dst(i, j);
            dst(i, j) = (float)(old + (double)factAB * s);
        }
}

}  // namespace cuv_oracle
#endif
