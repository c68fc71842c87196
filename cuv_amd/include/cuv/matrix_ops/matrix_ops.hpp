// prod() and spmv() with a device DIA matrix operand.
//
// Mirrors the dev_memory_space specialisations of the reference
// (src/cuv/matrix_ops/matrix_ops.hpp:117-119,277-278; bodies in
// src/cuv/matrix_ops/spmv.cu:89-101,130-139,221-253): same signatures, same
// preconditions (each throws std::runtime_error with the stringified
// condition), results visible on return.  The work is done by
// cuvdia_spmm_f32 (hand-written HIP for gfx950); there is no CPU fallback in
// this header -- the host_memory_space twins are in cuv/matrix_ops/host_ops.hpp.
#ifndef __CUV_MATRIX_OPS_HPP__
#define __CUV_MATRIX_OPS_HPP__

#include <cuv/basics/dia_matrix.hpp>
#include <cuv/basics/tensor.hpp>

namespace cuv {

/// dst = factC*dst + factAB*op(A)*B for a column-major batch B.
/// transA: 'n' or 't'; transB must be 'n'.  factC == 0 never reads dst.
inline void prod(tensor<float, dev_memory_space, column_major> &dst,
                 const dia_matrix<float, dev_memory_space> &A,
                 const tensor<float, dev_memory_space, column_major> &B,
                 char transA = 'n', char transB = 'n',
                 const float &factAB = 1.f, const float &factC = 0.f)
{
    cuvAssert(dst.shape().size() == 2);
    cuvAssert(B.shape().size() == 2);
    cuvAssert(transB == 'n');
    cuvAssert(dst.shape()[1] == B.shape()[1]);
    cuvAssert(dst.ptr());
    cuvAssert(A.vec_ptr());
    cuvAssert(B.ptr());
    cuvAssert(transA == 'n' || transA == 't');
    if (transA == 't') {
        cuvAssert(A.w() == dst.shape()[0]);
        cuvAssert(A.h() == B.shape()[0]);
    } else {
        cuvAssert(A.h() == dst.shape()[0]);
        cuvAssert(A.w() == B.shape()[0]);
    }
    checkDiaCall(cuvdia_spmm_f32(A.descriptor(), A.vec().ptr(), B.ptr(), (long long)B.shape()[0], dst.ptr(),
                                 (long long)dst.shape()[0], (int)B.shape()[1], transA, factAB, factC, NULL),
                 "cuvdia_spmm_f32");
    cuvSafeCall(hipStreamSynchronize(NULL));
}

/// dst = factC*dst + factAv*op(A)*v.  As in the reference, v and dst may hold
/// several consecutive columns (size a multiple of the matrix dimension).
inline void spmv(tensor<float, dev_memory_space> &dst, const dia_matrix<float, dev_memory_space> &A,
                 const tensor<float, dev_memory_space> &v, char transA = 'n',
                 const float &factAv = 1.f, const float &factC = 0.f)
{
    cuvAssert(transA == 'n' || transA == 't');
    cuvAssert(dst.ptr());
    cuvAssert(v.ptr());
    cuvAssert(A.vec_ptr());
    const unsigned int n_out = transA == 't' ? A.w() : A.h();
    const unsigned int n_in = transA == 't' ? A.h() : A.w();
    cuvAssert(v.size() % n_in == 0);
    const unsigned int batch = v.size() / n_in;
    cuvAssert(dst.size() == batch * n_out);
    checkDiaCall(cuvdia_spmm_f32(A.descriptor(), A.vec().ptr(), v.ptr(), (long long)n_in, dst.ptr(),
                                 (long long)n_out, (int)batch, transA, factAv, factC, NULL),
                 "cuvdia_spmm_f32");
    cuvSafeCall(hipStreamSynchronize(NULL));
}

}  // namespace cuv
#endif
