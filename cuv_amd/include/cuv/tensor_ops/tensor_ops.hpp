// fill() and sequence(): the two nullary fills the DIA fixtures use
// (src/cuv/tensor_ops/tensor_ops.hpp:106-122, functors in
// src/cuv/tensor_ops/tensor_ops.cuh:244-283 of the reference).  sequence()
// counts 0, 1, 2, ... in memory order.
#ifndef __CUV_TENSOR_OPS_HPP__
#define __CUV_TENSOR_OPS_HPP__

#include <vector>

#include <cuv/basics/tensor.hpp>

namespace cuv {

template <class V, class L, class S>
void fill(tensor<V, host_memory_space, L> &v, const S &p)
{
    V *d = v.ptr();
    for (size_t i = 0, n = v.size(); i < n; ++i) d[i] = (V)p;
}
template <class V, class L>
void sequence(tensor<V, host_memory_space, L> &v)
{
    V *d = v.ptr();
    for (size_t i = 0, n = v.size(); i < n; ++i) d[i] = (V)i;
}
// Device fills are fixture set-up, not hot path: build on the host, copy once.
template <class V, class L, class S>
void fill(tensor<V, dev_memory_space, L> &v, const S &p)
{
    std::vector<V> h(v.size(), (V)p);
    detail::copy<V, dev_memory_space, host_memory_space>(v.ptr(), h.data(), h.size());
}
template <class V, class L>
void sequence(tensor<V, dev_memory_space, L> &v)
{
    std::vector<V> h(v.size());
    for (size_t i = 0; i < h.size(); ++i) h[i] = (V)i;
    detail::copy<V, dev_memory_space, host_memory_space>(v.ptr(), h.data(), h.size());
}

}  // namespace cuv
#endif
