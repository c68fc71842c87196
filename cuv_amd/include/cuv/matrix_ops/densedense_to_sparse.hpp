// densedense_to_dia(): C_dia = factC*C_dia + factAB*proj(A*B'), on the device.
//
// Mirrors src/cuv/matrix_ops/densedense_to_sparse.hpp:52-139 of the reference
// (device body src/cuv/matrix_ops/densedense_to_sparse.cu:253-308): the same
// 6-argument signature with a block descriptor, the same preconditions, results
// visible on return, with the documented contract that both factors apply.
// The descriptor classes keep their names and constructors; on the device the
// descriptor is the matrix's O(num_dia) run table instead of the reference's
// list of 16x16 blocks (densedense_to_sparse.cu:123-171).  The
// host_memory_space twin of densedense_to_dia is in cuv/matrix_ops/host_ops.hpp.
#ifndef __DENSEDENSE_TO_SPARSE_HPP__
#define __DENSEDENSE_TO_SPARSE_HPP__

#include <cuv/basics/dia_matrix.hpp>

namespace cuv {

/// Does nothing; exists so host and device code share one call shape.
template <class __value_type, class __index_type = unsigned int>
class host_block_descriptor {
  public:
    typedef __value_type value_type;
    typedef __index_type index_type;
    typedef dia_matrix<value_type, host_memory_space, index_type> diamat_type;
    host_block_descriptor(const diamat_type &) {}
};

/// Pins the run table of a device DIA matrix; reusable for every matrix with
/// the same shape and offsets.
template <class __value_type, class __index_type = unsigned int>
class dev_block_descriptor {
  public:
    typedef __value_type value_type;
    typedef __index_type index_type;
    typedef dia_matrix<value_type, dev_memory_space, index_type> diamat_type;

  protected:
    const cuvdia_desc *m_desc;
    int m_len;
    int m_h, m_w, m_stride, m_rf;
    std::vector<int> m_offsets;

  public:
    dev_block_descriptor(const diamat_type &d)
        : m_desc(d.descriptor()), m_len(0), m_h(d.h()), m_w(d.w()), m_stride(d.stride()), m_rf(d.row_fact()),
          m_offsets(d.host_offsets())
    {
        checkDiaCall(cuvdia_desc_info(m_desc, &m_len, NULL, NULL), "cuvdia_desc_info");
    }
    ~dev_block_descriptor() {}
    /// number of run chunks (the reference returned its number of 16x16 blocks)
    inline int len() const { return m_len; }
    inline bool matches(const diamat_type &d) const
    {
        return m_h == (int)d.h() && m_w == (int)d.w() && m_stride == (int)d.stride() && m_rf == d.row_fact() &&
               m_offsets == d.host_offsets();
    }
};

template <class __memory_layout_type, class __index_type>
void densedense_to_dia(dia_matrix<float, dev_memory_space, __index_type> &C,
                       const dev_block_descriptor<float, __index_type> &Cbd,
                       const tensor<float, dev_memory_space, __memory_layout_type> &A,
                       const tensor<float, dev_memory_space, __memory_layout_type> &B,
                       const float &factAB = 1.f, const float &factC = 0.f)
{
    static_assert(std::is_same<__memory_layout_type, column_major>::value,
                  "densedense_to_dia takes column-major dense operands");
    cuvAssert(A.shape().size() == 2);
    cuvAssert(B.shape().size() == 2);
    cuvAssert(Cbd.matches(C));
    cuvAssert(C.vec_ptr());
    cuvAssert(C.w() == B.shape()[0]);
    cuvAssert(C.h() == A.shape()[0]);
    cuvAssert(A.shape()[1] == B.shape()[1]);
    checkDiaCall(cuvdia_dd2dia_f32(C.descriptor(), C.vec().ptr(), A.ptr(), (long long)A.shape()[0], B.ptr(),
                                   (long long)B.shape()[0], (int)A.shape()[1], factAB, factC, NULL),
                 "cuvdia_dd2dia_f32");
    cuvSafeCall(hipStreamSynchronize(NULL));
}

/// Convenience form without a descriptor argument (the matrix carries its own).
template <class __memory_layout_type, class __index_type>
void densedense_to_dia(dia_matrix<float, dev_memory_space, __index_type> &C,
                       const tensor<float, dev_memory_space, __memory_layout_type> &A,
                       const tensor<float, dev_memory_space, __memory_layout_type> &B,
                       const float &factAB = 1.f, const float &factC = 0.f)
{
    dev_block_descriptor<float, __index_type> bd(C);
    densedense_to_dia(C, bd, A, B, factAB, factC);
}

}  // namespace cuv
#endif
