// avg_diagonals(): the mean of every stored diagonal of a device DIA matrix.
//
// Mirrors src/cuv/matrix_ops/diagonals.hpp:12 of the reference (bodies in
// src/cuv/matrix_ops/diagonals.cu:8-61) for dev_memory_space: same signature,
// the preconditions of the host version (diagonals.cu:28-29), result visible
// on return.  The mean runs over the valid slots of a diagonal, as in the
// reference's host version; padding is never read.  The host_memory_space
// twin is in cuv/matrix_ops/host_ops.hpp.
#ifndef __CUV_DIAGONALS_HPP__
#define __CUV_DIAGONALS_HPP__

#include <cuv/basics/dia_matrix.hpp>
#include <cuv/basics/tensor.hpp>

namespace cuv {

/// dst[i] = mean of the diagonal at table position i.
inline void avg_diagonals(tensor<float, dev_memory_space> &dst, const dia_matrix<float, dev_memory_space> &dia)
{
    cuvAssert(dia.row_fact() == 1);
    cuvAssert((size_t)dia.num_dia() == (size_t)dst.size());
    cuvAssert(dst.ptr());
    cuvAssert(dia.vec_ptr());
    checkDiaCall(cuvdia_avg_diagonals_f32(dia.descriptor(), dia.vec().ptr(), dst.ptr(), NULL),
                 "cuvdia_avg_diagonals_f32");
    cuvSafeCall(hipStreamSynchronize(NULL));
}

}  // namespace cuv
#endif
