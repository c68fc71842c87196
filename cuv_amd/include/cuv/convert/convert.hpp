// convert(dst, src) for the DIA path: dense host<->device copies of equal
// layout, DIA host<->device, and DIA -> dense on the host.
//
// Mirrors src/cuv/convert/convert.cu:42-112,131-137,222-245 of the reference:
// the destination is re-allocated when its shape (or row_fact, or a missing
// value vector) does not match the source; DIA copies move the offset table
// and the value vector and rebuild the offset map; DIA -> dense zero-fills and
// walks each stored diagonal.
#ifndef __CUV_CONVERT_HPP__
#define __CUV_CONVERT_HPP__

#include <algorithm>

#include <cuv/basics/dia_matrix.hpp>
#include <cuv/basics/tensor.hpp>

namespace cuv {

// dense, same value type and layout, any pair of memory spaces
template <class V, class MD, class MS, class L>
void convert(tensor<V, MD, L> &dst, const tensor<V, MS, L> &src)
{
    if (dst.shape() != src.shape()) {
        tensor<V, MD, L> d(src.shape());
        dst = d;
    }
    detail::copy<V, MD, MS>(dst.ptr(), src.ptr(), src.size());
}

// DIA, host <-> device (either direction, or same space)
template <class V, class MD, class MS, class I>
void convert(dia_matrix<V, MD, I> &dst, const dia_matrix<V, MS, I> &src)
{
    if (dst.shape()[0] != src.shape()[0] || dst.shape()[1] != src.shape()[1] ||
        dst.row_fact() != src.row_fact() || dst.num_dia() != src.num_dia() ||
        dst.stride() != src.stride() || !dst.vec_ptr()) {
        dst.dealloc();
        dst = dia_matrix<V, MD, I>(src.shape()[0], src.shape()[1], src.num_dia(), src.stride(), src.row_fact());
    }
    cuvAssert(dst.vec_ptr());
    cuvAssert(src.vec_ptr());
    cuvAssert(dst.get_offsets().ptr());
    cuvAssert(dst.vec().ptr());
    dst.set_offsets(src.host_offsets());
    detail::copy<V, MD, MS>(dst.vec().ptr(), src.vec().ptr(), src.vec().size());
}

// DIA -> dense, host
template <class V, class L, class I>
void convert(tensor<V, host_memory_space, L> &dst, const dia_matrix<V, host_memory_space, I> &src)
{
    if (dst.ndim() != 2 || dst.shape()[0] != src.shape()[0] || dst.shape()[1] != src.shape()[1]) {
        tensor<V, host_memory_space, L> d(src.shape()[0], src.shape()[1]);
        dst = d;
    }
    fill(dst, 0);
    const std::vector<int> &off = src.host_offsets();
    const int rf = src.row_fact();
    for (unsigned int oi = 0; oi < off.size(); oi++) {
        const int o = off[oi];
        I j = (I)std::max(0, o);
        I i = (I)(rf * std::max(0, -o));
        for (; i < src.shape()[0] && j < src.shape()[1]; j++)
            for (int k = 0; k < rf && i < src.shape()[0]; k++, i++) dst(i, j) = src(i, j);
    }
}

}  // namespace cuv
#endif
